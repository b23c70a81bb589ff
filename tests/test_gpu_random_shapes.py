"""Seeded random shapes, layouts, split counts and scratch on/off through the library's own choice of kernel,
against the exact oracle: the dispatch rules (tile shape by tile count, automatic and explicit splits with uneven
parts, scale staging, streaming kernel) are exercised at shapes nobody picked by hand."""

import os

import numpy as np
import pytest
import torch

import wave_amd

from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import assert_close, run_gemm

pytestmark = pytest.mark.gpu


def _cases(count, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        kind = rng.integers(0, 4)
        if kind == 0:    # decode-like
            m, n, k = int(rng.integers(1, 65)), int(rng.integers(1, 3000)), 32 * int(rng.integers(1, 160))
        elif kind == 1:  # small and ragged
            m, n, k = int(rng.integers(1, 400)), int(rng.integers(1, 400)), 32 * int(rng.integers(1, 64))
        elif kind == 2:  # few tiles, long K (automatic split)
            m, n, k = int(rng.integers(65, 700)), int(rng.integers(100, 700)), 256 * int(rng.integers(8, 40))
        else:            # many tiles, short K
            m, n, k = int(rng.integers(500, 2200)), int(rng.integers(500, 2200)), 32 * int(rng.integers(4, 24))
        out.append((i, m, n, k, int(rng.integers(0, 3)), int(rng.integers(0, 3)), bool(rng.integers(0, 2)),
                    bool(rng.integers(0, 2)), bool(rng.integers(0, 4) > 0)))
    return out


@pytest.mark.parametrize("case", _cases(48, seed=20), ids=lambda c: f"{c[0]}-{c[1]}x{c[2]}x{c[3]}")
def test_random_shape_against_oracle(case):
    i, m, n, k, a_layout, b_layout, preshuffle, bf16, scratch = case
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=1000 + i, scale_lo=118, scale_hi=136)
    rows = np.unique(np.r_[0:min(m, 4), m // 2, max(0, m - 3):m])
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    layouts = [_lib.SCALE_ROW_MAJOR, _lib.SCALE_E8M0_SHUFFLE, _lib.SCALE_MFMA32]
    conv = {_lib.SCALE_ROW_MAJOR: lambda s: s, _lib.SCALE_E8M0_SHUFFLE: orc.e8m0_shuffle_padded,
            _lib.SCALE_MFMA32: orc.mfma32_scale_layout}
    kw = dict(a_scale_layout=layouts[a_layout], b_scale_layout=layouts[b_layout])
    if preshuffle and n % 16 == 0 and k % 64 == 0:
        w_in, kw["b_layout"] = orc.b_preshuffle(w_t), _lib.B_PRESHUFFLE
    else:
        w_in = w_t
    if not scratch:
        kw["workspace"] = False
    out_dtype = torch.bfloat16 if bf16 else torch.float32
    got = run_gemm(x, conv[layouts[a_layout]](xs), w_in, conv[layouts[b_layout]](ws), out_dtype, **kw)
    assert not np.isnan(got).any()
    assert_close(got[rows], ref, out_dtype, f"case {case}")


def _wide_cases(count, seed):
    """Shapes the newer kernels take under the library's own choice: up to 256 rows against a wide N (mid-M kernel,
    every strip width and block shape, K with and without the rotated start), more than 256 tiles with N a multiple of 192 (256x192 tiles) or with preshuffled B
    (B-direct kernel), K a multiple of 256 so that they qualify, and ragged M."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        kind = rng.integers(0, 3)
        if kind == 0:    # mid-M
            m, n, k = int(rng.integers(1, 257)), 4 * int(rng.integers(3072, 9000)), 256 * int(rng.integers(4, 17))
        elif kind == 1:  # 256x192 tiles
            m, n, k = int(rng.integers(2100, 5000)), 192 * int(rng.integers(20, 40)), 256 * int(rng.integers(3, 8))
        else:            # more tiles than CUs, N % 256 == 0 (B-direct when preshuffled)
            m, n, k = int(rng.integers(2100, 5000)), 256 * int(rng.integers(14, 24)), 512 * int(rng.integers(3, 6))
        out.append((i, m, n, k, int(rng.integers(0, 3)), int(rng.integers(0, 3)), bool(rng.integers(0, 2)),
                    bool(rng.integers(0, 2)), bool(rng.integers(0, 4) > 0)))
    return out


@pytest.mark.parametrize("case", _wide_cases(18, seed=21), ids=lambda c: f"w{c[0]}-{c[1]}x{c[2]}x{c[3]}")
def test_random_wide_shape_against_oracle(case):
    test_random_shape_against_oracle(case)


def _midb_cases(count, seed):
    """Shapes the library's own choice gives to the B-direct mid-M kernel when B is preshuffled (128 < M <= 256,
    N >= 12288 in whole 32-column tiles, K in whole turns of its ring), with every scale layout and with and
    without scratch (without it, and with scales that are not in MFMA32 order, the strip kernel takes them)."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        m, n, k = int(rng.integers(129, 257)), 32 * int(rng.integers(384, 1000)), 1024 * int(rng.integers(1, 9))
        out.append((i, m, n, k, int(rng.integers(0, 3)), int(rng.integers(0, 3)), True, bool(rng.integers(0, 2)),
                    bool(rng.integers(0, 4) > 0)))
    return out


@pytest.mark.parametrize("case", _midb_cases(int(os.environ.get("WAVE_MIDB_FUZZ", "10")), seed=22),
                         ids=lambda c: f"b{c[0]}-{c[1]}x{c[2]}x{c[3]}")
def test_random_preshuffled_mid_shape_against_oracle(case):
    test_random_shape_against_oracle(case)


def _resident_cases(count, seed):
    """Shapes on either side of the borders the library's own choice follows when both scale tensors come in MFMA32
    order (streaming kernel, mid-M kernel, 128x128 tiles, B-direct mid-M kernel from 32 rows on with a preshuffled
    B): up to 256 rows, N from 12288 to past one round of 128-column strips, K = 2048 / 4096 / 8192."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        m = int(rng.choice([rng.integers(1, 17), rng.integers(17, 65), rng.integers(65, 129), rng.integers(129, 257)]))
        n = 32 * int(rng.choice([rng.integers(384, 513), rng.integers(513, 1025), rng.integers(1025, 1400)]))
        k = int(rng.choice([2048, 4096, 8192]))
        out.append((i, m, n, k, 2, 2, bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 4) > 0)))
    return out


@pytest.mark.parametrize("case", _resident_cases(12, seed=23), ids=lambda c: f"r{c[0]}-{c[1]}x{c[2]}x{c[3]}")
def test_random_resident_scale_shape_against_oracle(case):
    test_random_shape_against_oracle(case)


@pytest.mark.parametrize("m,n,k", [(33, 512, 8192), (48, 3000, 8192), (64, 1024, 14336), (64, 4096, 8192), (40, 3072, 16384),
                                   (64, 4100, 8192), (32, 1024, 8192)])
def test_narrow_b_long_k_against_oracle(m, n, k):
    """32 < M <= 64 against a B of at most 4096 rows with K > 4096: the library's own choice is the 128x128 tiles
    with its split along K (the last two cases lie just outside that range: the streaming kernel).  Every row
    against the exact oracle, both output types, with and without scratch."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + n, scale_lo=120, scale_hi=134)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    for dt in (torch.float32, torch.bfloat16):
        for kw in ({}, {"workspace": False}):
            got = run_gemm(x, xs, w_t, ws, dt, **kw)
            assert not np.isnan(got).any()
            assert_close(got, ref, dt, f"{m}x{n}x{k} {dt} {kw}")


@pytest.mark.parametrize("m,n,k", [(1, 8192, 9216), (16, 8448, 11008), (16, 4096, 14080), (64, 2048, 12032),
                                   (8, 12288, 6400), (16, 4096, 6400), (5, 8192, 13824), (33, 8192, 14080),
                                   (1, 4096, 11008), (8, 8192, 11008), (32, 6144, 11008), (64, 6144, 8192)])
def test_decode_rows_with_uneven_k_tiles_against_oracle(m, n, k):
    """Up to 64 rows with a count of K tiles that the streaming kernel cannot deal evenly over its waves (25, 36, 43,
    47, 54 and 55 tiles: the K of Llama-2 down projections among them): the library's own choice is the mid-M
    kernel against a wide B and the 128x128 tiles with a split along K against a narrow one (the last four: the
    direct whole-K kernel for a prime count of K tiles at few rows, and the mid-M kernel from N = 6144 on).  Every
    row against the exact oracle, both output types, with and without scratch."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=120, scale_hi=134)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    for dt in (torch.float32, torch.bfloat16):
        for kw in ({}, {"workspace": False}):
            got = run_gemm(x, xs, w_t, ws, dt, **kw)
            assert not np.isnan(got).any()
            assert_close(got, ref, dt, f"{m}x{n}x{k} {dt} {kw}")


@pytest.mark.parametrize("m,n,k", [(2773, 1408, 1024), (3300, 1152, 2304), (5600, 640, 1280)])
def test_half_empty_last_column_tile_against_oracle(m, n, k):
    """An N that leaves the last 256-column tile half empty, with more than 128 tiles of 128x256 but at most 256 of
    128x128: the library's own choice is the latter.  Sampled rows against the exact oracle, the whole output
    against the 128x128 tiles by name (the same K order per element: the same bits)."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + n, scale_lo=120, scale_hi=134)
    rows = np.unique(np.concatenate([np.arange(0, m, 41), np.arange(m - 5, m)]))
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    for dt in (torch.float32, torch.bfloat16):
        got = run_gemm(x, xs, w_t, ws, dt)
        assert_close(got[rows], ref, dt, f"{m}x{n}x{k} {dt}")
        assert np.array_equal(got, run_gemm(x, xs, w_t, ws, dt, variant=_lib.VARIANT_T128x128_W2x2))


@pytest.mark.parametrize("m,n,k", [(176, 3200, 8960), (97, 8832, 15616), (76, 4480, 13312), (384, 3584, 8192),
                                   (134, 6272, 12032), (768, 3584, 11008), (1280, 3584, 4096), (256, 11008, 4096)])
def test_estimated_tile_shape_and_split_against_oracle(m, n, k):
    """Problems of at most two rounds of 256x256 tiles, where the library's own choice of tile shape and split comes
    from its duration estimates: splits into 3, 5 and 7 uneven parts on the 128x128 and 128x256 tiles, a problem of
    280 tiles of 128x128 with a short K (scales re-laid, not staged by the kernel), and one for the mid-M kernel.
    Sampled rows against the exact oracle with row-major scales and with scales in MFMA32 order, both output types,
    and without scratch (no split then)."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=120, scale_hi=134)
    rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 24)), np.arange(m - 4, m)]))
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    xs32 = wave_amd.scale_convert(torch.from_numpy(xs).cuda(), m, k // 32, 0, _lib.SCALE_MFMA32).cpu().numpy()
    ws32 = wave_amd.scale_convert(torch.from_numpy(ws).cuda(), n, k // 32, 0, _lib.SCALE_MFMA32).cpu().numpy()
    for dt in (torch.float32, torch.bfloat16):
        got = run_gemm(x, xs, w_t, ws, dt)
        assert not np.isnan(got).any()
        assert_close(got[rows], ref, dt, f"{m}x{n}x{k} {dt} row-major scales")
        got = run_gemm(x, xs32, w_t, ws32, dt, a_scale_layout=_lib.SCALE_MFMA32, b_scale_layout=_lib.SCALE_MFMA32)
        assert not np.isnan(got).any()
        assert_close(got[rows], ref, dt, f"{m}x{n}x{k} {dt} MFMA32 scales")
    got = run_gemm(x, xs, w_t, ws, torch.float32, workspace=False)
    assert_close(got[rows], ref, torch.float32, f"{m}x{n}x{k} without scratch")
