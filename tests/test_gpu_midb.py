"""GPU: the B-direct mid-M kernel (variant 10: 64 < M <= 256 against a wide preshuffled B, A through an LDS ring,
B straight from global memory into registers; the reference's asymmetric data flow,
wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:950-991) against the exact oracle: both block heights, ragged
M, N ending inside a strip, a K walk that starts at every K tile, both output types, every scale layout, NaN scales,
and the library's own choice of it."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu
V = _lib.VARIANT_MID_M_BDIRECT


def run(x, xs, w, ws, dt, **kw):
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    gwp = wave_amd.b_preshuffle(gw)
    out = torch.full((x.shape[0], w.shape[0]), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gwp, gws, out, b_layout=_lib.B_PRESHUFFLE, **kw)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [
    (128, 128, 2048),    # one strip, the 128-row block, one turn of its ring of 8 K tiles
    (256, 128, 1024),    # the 256-row block, one turn of its ring of 4
    (65, 512, 4096),     # ragged M below a block
    (100, 1056, 2048),   # N ends inside a strip (32 of its 128 columns)
    (129, 384, 3072),    # just above 128 rows: the 256-row block (K in turns of 4 K tiles)
    (200, 2048, 8192),   # 16 strips
    (256, 4096, 2048),   # 32 strips: workgroups 0, 8, 16, 24 of an XCD start at K tiles 0 .. 3
    (1, 256, 2048),      # a single row by name
])
def test_midb_small_shapes_whole_oracle(m, n, k, dt):
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + n + k, scale_lo=110, scale_hi=140)
    ref = c_oracle.scaled_gemm_exact(x, w, xs, ws)
    assert_close(run(x, xs, w, ws, dt, variant=V, split_k=1), ref, dt, f"{m}x{n}x{k}")


@pytest.mark.parametrize("m,k", [(128, 2048), (192, 1024)])
def test_midb_every_start_of_the_k_walk(m, k):
    """Workgroup w starts at K tile (w / 8) mod K tiles: with 8 * K tiles strips every start occurs, the walk wraps
    around the end of K at every position, and the requests past its end are dropped at every position."""
    n = 128 * 8 * (k // 256)
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=k + m, scale_lo=100, scale_hi=154)
    ref = c_oracle.scaled_gemm_exact(x, w, xs, ws)
    assert_close(run(x, xs, w, ws, torch.float32, variant=V, split_k=1), ref, torch.float32, f"{m}x{n}x{k}")


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m", [96, 128, 160, 256])
def test_midb_decode_shape(m, dt):
    """The shape the kernel is for (N = 28672, K = 8192: 224 strips): rows of every 32-row block against the oracle,
    every element against the strip kernel for row-major B (same sums in another order: tolerance, not bits)."""
    n, k = 28672, 8192
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=2 + m, scale_lo=120, scale_hi=134)
    c = run(x, xs, w, ws, dt, variant=V, split_k=1)
    rows = np.unique(np.concatenate([np.arange(0, m, 7), [m - 1]]))
    assert_close(c[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), dt, "rows vs oracle")
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    other = torch.empty(m, n, dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, other, variant=_lib.VARIANT_MID_M, split_k=1)
    assert_close(c, other.float().cpu().numpy().astype(np.float64), dt, "all elements vs the strip kernel")


def test_midb_scale_layouts_and_auto_choice():
    m, n, k = 160, 14336, 4096
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=9, scale_lo=100, scale_hi=154)
    forced = run(x, xs, w, ws, torch.float32, variant=V, split_k=1)
    assert_close(forced, c_oracle.scaled_gemm_exact(x, w, xs, ws), torch.float32, "oracle")
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    gwp = wave_amd.b_preshuffle(gw)
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    # the library's own choice for a preshuffled B of this shape
    wave_amd.mxfp4_gemm(gx, gxs, gwp, gws, out, b_layout=_lib.B_PRESHUFFLE)
    assert np.array_equal(out.cpu().numpy(), forced)
    # scales handed over in e8m0_shuffle order and in MFMA32 order (no re-layout launch, no scratch): the same bits
    xs_sh, ws_sh = wave_amd.e8m0_shuffle(gxs), wave_amd.e8m0_shuffle(gws)
    wave_amd.mxfp4_gemm(gx, xs_sh, gwp, ws_sh, out, b_layout=_lib.B_PRESHUFFLE, variant=V, split_k=1,
                        a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert np.array_equal(out.cpu().numpy(), forced)
    xs32 = wave_amd.scale_convert(gxs, m, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32)
    ws32 = wave_amd.scale_convert(gws, n, k // 32, _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32)
    wave_amd.mxfp4_gemm(gx, xs32, gwp, ws32, out, b_layout=_lib.B_PRESHUFFLE, variant=V, split_k=1,
                        a_scale_layout=_lib.SCALE_MFMA32, b_scale_layout=_lib.SCALE_MFMA32, workspace=False)
    assert np.array_equal(out.cpu().numpy(), forced)


def test_midb_nan_scale_poisons_its_row_and_column():
    m, n, k = 160, 512, 2048
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=5, scale_lo=120, scale_hi=134)
    xs[100, 17] = 255
    ws[77, 63] = 255
    c = run(x, xs, w, ws, torch.float32, variant=V, split_k=1)
    ref = c_oracle.scaled_gemm_exact(x, w, xs, ws)
    assert np.isnan(c[100]).all() and np.isnan(c[:, 77]).all()
    assert_close(c, ref, torch.float32, "NaN scales")


def test_midb_refuses_what_it_does_not_take():
    x, xs, w, ws = orc.make_inputs(128, 256, 1536, seed=1)   # K not in whole turns of the ring
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    out = torch.empty(128, 256, dtype=torch.float32, device=DEV)
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(gx, gxs, wave_amd.b_preshuffle(gw), gws, out, b_layout=_lib.B_PRESHUFFLE, variant=V, split_k=1)
    x, xs, w, ws = orc.make_inputs(128, 256, 2048, seed=1)   # row-major B
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, variant=V, split_k=1)
