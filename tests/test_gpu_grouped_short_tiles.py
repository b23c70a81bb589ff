"""GPU: short tiles of the grouped persistent kernel.  A group's last 256-row M tile of at most 64 rows runs after
all full tiles, with the eight waves side by side on its 64 rows (wave_amd/csrc/mxfp4_gemm_persist.hip), in place
of the per-expert loop of the reference's MoE tests (tests/kernel/moe_test.py:175-246), whose groups are as ragged.

Cases: groups of 1, 63, 64, 65 and 257 rows beside large and empty ones; nothing but short tiles (every workgroup
starts with one); no short tile at all; both output types; scales row-major and already in MFMA32 order.  Rows of
every group against the exact oracle, every element against the one-tile-per-workgroup kernel."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu


def inputs(counts, n, k, seed):
    rows = int(sum(counts))
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    x, xs, _, _ = orc.make_inputs(rows, 1, k, seed, scale_lo=118, scale_hi=136)
    rng = np.random.default_rng(seed + 100)
    e = len(counts)
    w = rng.integers(0, 256, size=(e, n, k // 2), dtype=np.uint8)
    ws = rng.integers(118, 137, size=(e, n, k // 32), dtype=np.uint8)
    return x, xs, w, ws, off


def run_and_check(counts, n, k, dt, seed, native_scales=False):
    x, xs, w, ws, off = inputs(counts, n, k, seed)
    rows, e = x.shape[0], len(counts)
    gx, gxs, gw, gws, goff = to_gpu(x, xs, w, ws, off)
    kw = {}
    a_s, b_s = gxs, gws
    if native_scales:
        a_s = wave_amd.scale_convert(gxs, rows, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32)
        b_s = torch.stack([wave_amd.scale_convert(gws[g], n, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32) for g in range(e)])
        kw = dict(a_scale_layout=_lib.SCALE_MFMA32, b_scale_layout=_lib.SCALE_MFMA32)
    out = torch.full((rows + 3, n), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, a_s, gw, b_s, goff, out[:rows], variant=_lib.VARIANT_T256x256_W4x2, **kw)
    torch.cuda.synchronize()
    c = out.float().cpu().numpy()
    assert np.isnan(c[rows:]).all(), "rows past the last offset were written"
    assert not np.isnan(c[:rows]).any(), "elements left unwritten"
    for g in range(e):
        lo, hi = int(off[g]), int(off[g + 1])
        if hi == lo:
            continue
        pick = np.unique(np.concatenate([np.arange(lo, hi, 53), np.arange(lo + 255, hi, 256), np.arange(lo, hi, 256),
                                         np.arange(max(lo, hi - 3), hi)]))
        ref = c_oracle.scaled_gemm_exact(x, w[g], xs, ws[g], rows=pick)
        assert_close(c[pick], ref, dt, f"group {g} ({hi - lo} rows)")
    other = torch.full((rows, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, other, variant=_lib.VARIANT_T128x128_W2x2, workspace=False)
    torch.cuda.synchronize()
    o = other.cpu().numpy()
    assert np.abs(c[:rows] - o).max() <= (4e-6 if dt == torch.float32 else 2.0 ** -7) * np.abs(o).max()


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("native", [False, True])
def test_groups_of_1_63_64_65_257_rows_beside_large_ones(dt, native):
    # tiles: 1 (short), 1 (short), 1 (short), 1 (full: 65 rows), 2 (256 full + 1 short), 6 (5 full + 220 rows full),
    # none, 10 (9 full + 196 rows full) x 16 columns = 272 full + 64 short on 256 workgroups
    run_and_check([1, 63, 64, 65, 257, 1500, 0, 2500], 4096, 1024, dt, seed=31, native_scales=native)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_nothing_but_short_tiles(dt):
    # 80 groups of at most 64 rows (one of none), 32 columns of tiles: 2528 short tiles, no full one; every
    # workgroup starts with a short tile
    rng = np.random.default_rng(5)
    counts = [int(c) for c in rng.integers(1, 65, 80)]
    counts[7] = 0
    counts[11] = 64
    assert sum(counts) // 256 * 32 > 256
    run_and_check(counts, 8192, 768, dt, seed=32)


def test_few_full_tiles_then_short_ones():
    # 10 full tiles x 32 columns = 320 ids over 256 workgroups, then 12 groups' short tiles: some workgroups run
    # full, full, short; some full, short; and the padding ids between the two parts of the walk are skipped
    run_and_check([1280, 1281, 30, 40, 50, 60, 7, 8, 9, 10, 11, 12, 13, 64], 8192, 1024, torch.bfloat16, seed=33)


def test_no_short_tile_at_all():
    run_and_check([1024, 1000, 2048, 200, 65, 300], 4096, 1024, torch.float32, seed=34)
