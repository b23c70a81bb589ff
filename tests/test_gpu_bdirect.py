"""GPU: the B-direct kernel (variant 7: A through LDS, preshuffled B straight from global memory into registers,
the reference's asymmetric family, wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:950-991) against the exact
oracle: single tile, ragged M, several tiles per workgroup (more tiles than CUs), both output types, all scale
layouts, and the library's own choice of it for preshuffled B."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu
V = _lib.VARIANT_T256x256_W1x4_BDIRECT


def run(x, xs, w, ws, dt, **kw):
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    gwp = wave_amd.b_preshuffle(gw)
    out = torch.full((x.shape[0], w.shape[0]), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gwp, gws, out, b_layout=_lib.B_PRESHUFFLE, **kw)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(256, 256, 1536), (1, 256, 2048), (300, 512, 2048), (1024, 1024, 4096),
                                   (77, 768, 8192), (513, 256, 3072)])
def test_bdirect_small_shapes_whole_oracle(m, n, k, dt):
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=110, scale_hi=140)
    ref = c_oracle.scaled_gemm_exact(x, w, xs, ws)
    assert_close(run(x, xs, w, ws, dt, variant=V, split_k=1), ref, dt, f"{m}x{n}x{k}")


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(4352, 4096, 1536), (4093, 6144, 3072)])
def test_bdirect_more_tiles_than_cus(m, n, k, dt):
    """272 and 384 tiles on 256 CUs: workgroups walk two tiles, the request streams run across the boundary; the
    last workgroups' second tile lies past M.  Rows of every M tile against the oracle, every element against the
    symmetric persistent kernel (same sums in a different order: tolerance, not bits)."""
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=118, scale_hi=136)
    c = run(x, xs, w, ws, dt, variant=V, split_k=1)
    rows = np.unique(np.concatenate([np.arange(0, m, 29), [m - 1, m - 2, 255, 256]]))
    assert_close(c[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), dt, "rows vs oracle")
    other = run(x, xs, w, ws, dt, variant=_lib.VARIANT_T256x256_W4x2, split_k=1)
    assert_close(c, other.astype(np.float64), dt, "all elements vs the symmetric kernel")


def test_bdirect_scale_layouts_and_auto_choice():
    m, n, k = 4608, 4096, 2048            # 288 tiles > 256 CUs: AUTO takes the B-direct kernel for preshuffled B
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=9, scale_lo=100, scale_hi=154)
    forced = run(x, xs, w, ws, torch.float32, variant=V, split_k=1)
    rows = np.unique(np.concatenate([np.arange(0, m, 41), [m - 1]]))
    assert_close(forced[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), torch.float32, "rows vs oracle")
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    gwp = wave_amd.b_preshuffle(gw)
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    # the library's own choice (split_k = 1: the K cut of a sparse last round belongs to the symmetric kernel)
    wave_amd.mxfp4_gemm(gx, gxs, gwp, gws, out, b_layout=_lib.B_PRESHUFFLE, split_k=1)
    assert np.array_equal(out.cpu().numpy(), forced)
    # scales handed over in e8m0_shuffle order and in MFMA32 order (no re-layout launch): the same bits
    xs_sh, ws_sh = wave_amd.e8m0_shuffle(gxs), wave_amd.e8m0_shuffle(gws)
    wave_amd.mxfp4_gemm(gx, xs_sh, gwp, ws_sh, out, b_layout=_lib.B_PRESHUFFLE, variant=V, split_k=1,
                        a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert np.array_equal(out.cpu().numpy(), forced)
    xs32 = wave_amd.scale_convert(gxs, m, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32)
    ws32 = wave_amd.scale_convert(gws, n, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32)
    wave_amd.mxfp4_gemm(gx, xs32, gwp, ws32, out, b_layout=_lib.B_PRESHUFFLE, variant=V, split_k=1,
                        a_scale_layout=_lib.SCALE_MFMA32, b_scale_layout=_lib.SCALE_MFMA32, workspace=False)
    assert np.array_equal(out.cpu().numpy(), forced)


def test_bdirect_nan_scale_poisons_its_row_and_column():
    m, n, k = 512, 512, 2048
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=5, scale_lo=120, scale_hi=134)
    xs[300, 17] = 255
    ws[77, 63] = 255
    c = run(x, xs, w, ws, torch.float32, variant=V, split_k=1)
    ref = c_oracle.scaled_gemm_exact(x, w, xs, ws)
    assert np.isnan(c[300]).all() and np.isnan(c[:, 77]).all()
    assert_close(c, ref, torch.float32, "NaN scales")
