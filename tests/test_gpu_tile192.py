"""GPU: the persistent kernel on 256x192 tiles (variant 9: the library's own choice when tiles of 256x256 would
leave the last round over the CUs partly empty; the reference fixes one block shape per compiled kernel,
wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:38-145) against the exact oracle and the 256x256 kernel:
ragged M, a partial last K tile, both output types (bf16 takes a narrower last pass through the C staging for the
wave's third 32-column tile), scale layouts, and the shapes AUTO takes it for."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu
V = _lib.VARIANT_T256x192_W4x2


def run(x, xs, w, ws, dt, **kw):
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    out = torch.full((x.shape[0], w.shape[0]), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, **kw)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(4093, 6144, 1024), (4352, 3840, 1536), (8192, 6336, 768), (4100, 3840, 1184)])
def test_tile192_rows_vs_oracle_and_all_vs_256(m, n, k, dt):
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=110, scale_hi=142)
    c = run(x, xs, w, ws, dt, variant=V, split_k=1)
    rows = np.unique(np.concatenate([np.arange(0, m, 37), np.arange(m - 40, m), [255, 256]]))
    assert_close(c[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), dt, "rows vs oracle")
    other = run(x, xs, w, ws, dt, variant=_lib.VARIANT_T256x256_W4x2, split_k=1)
    # the same K order per element in both tile shapes: the same bits
    assert np.array_equal(c, other)


def test_tile192_auto_choice_and_scale_layouts():
    m, n, k = 4093, 6144, 1024            # 384 tiles of 256x256 = 1.5 rounds of 256 CUs; 512 of 256x192 = 2
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=4, scale_lo=100, scale_hi=154)
    forced = run(x, xs, w, ws, torch.float32, variant=V, split_k=1)
    assert np.array_equal(run(x, xs, w, ws, torch.float32), forced)
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm(gx, wave_amd.e8m0_shuffle(gxs), gw, wave_amd.e8m0_shuffle(gws), out, variant=V, split_k=1,
                        a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert np.array_equal(out.cpu().numpy(), forced)
    wp = wave_amd.b_preshuffle(gw)
    wave_amd.mxfp4_gemm(gx, gxs, wp, gws, out, variant=V, split_k=1, b_layout=_lib.B_PRESHUFFLE)
    assert np.array_equal(out.cpu().numpy(), forced)


def test_tile192_rejects_what_it_does_not_take():
    x, xs, w, ws = orc.make_inputs(512, 768, 1024, seed=1)       # 8 tiles: not more than the CUs
    with pytest.raises((RuntimeError, ValueError)):
        run(x, xs, w, ws, torch.float32, variant=V, split_k=1)
    x, xs, w, ws = orc.make_inputs(4352, 4096, 1024, seed=1)     # N % 192 != 0
    with pytest.raises((RuntimeError, ValueError)):
        run(x, xs, w, ws, torch.float32, variant=V, split_k=1)


def test_tile192_auto_choice_where_n_is_not_in_whole_256_column_tiles():
    """N = 102 x 192 = 76.5 x 256: the 256x256 tiles would run one per workgroup in two whole rounds over the CUs
    (4 x 77 = 308 tiles), the library's own choice is the persistent kernel on 4 x 102 tiles of 256x192.  The same
    bits as that kernel by name, sampled rows against the exact oracle, and a shape of one round (3 x 77 tiles) that
    stays on the wider tiles."""
    m, n, k = 896, 19584, 1024
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=9, scale_lo=110, scale_hi=142)
    for dt in (torch.float32, torch.bfloat16):
        auto = run(x, xs, w, ws, dt)
        assert np.array_equal(auto, run(x, xs, w, ws, dt, variant=V, split_k=1))
        rows = np.unique(np.concatenate([np.arange(0, m, 61), np.arange(m - 8, m), [255, 256]]))
        assert_close(auto[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), dt, "rows vs oracle")
    m = 640
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=10, scale_lo=110, scale_hi=142)
    auto = run(x, xs, w, ws, torch.float32)
    rows = np.arange(0, m, 53)
    assert_close(auto[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), torch.float32, "one round")


@pytest.mark.parametrize("native", [False, True], ids=["row_major_scales", "mfma32_scales"])
def test_tile192_auto_choice_outside_the_range_of_the_duration_estimates(native):
    """K below the range where the library chooses by duration estimates, N = 30 x 192 = 22.5 x 256, 16 tile rows: the
    borders pick the 256x256 tiles, which would run in two whole rounds, and from there the persistent kernel on
    480 tiles of 256x192 - with either scale layout the same bits as that kernel by name."""
    m, n, k = 4096, 5760, 1024
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=12, scale_lo=110, scale_hi=142)
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    kw = {}
    if native:
        gxs = wave_amd.scale_convert(gxs, m, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32)
        gws = wave_amd.scale_convert(gws, n, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32)
        kw = dict(a_scale_layout=_lib.SCALE_MFMA32, b_scale_layout=_lib.SCALE_MFMA32)
    auto = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    named = torch.full_like(auto, float("nan"))
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, auto, **kw)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, named, variant=V, split_k=1, **kw)
    torch.cuda.synchronize()
    assert torch.equal(auto, named)
    rows = np.unique(np.concatenate([np.arange(0, m, 173), [255, 256, m - 1]]))
    assert_close(auto.cpu().numpy()[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), torch.float32, "rows vs oracle")
