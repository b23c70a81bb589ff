"""GPU: the large-tile persistent kernels reading both scale tensors in the reference's e8m0_shuffle order in
place (wave_lang/kernel/wave/utils/mxfp_utils.py:113-128; the reference's preshuffled-scale kernel families read
that format straight from global memory, wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:334-403,485-536).

The cases run without any workspace (with one the library re-lays the scales first, which is faster), so that no
re-layout pass can stand in for the in-place read, and are held to two bars: rows of every M tile against the exact oracle, and every element bit-equal to the same kernel fed the
same scales in MFMA32 order (the two differ only in how a lane finds its four scale bytes)."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu
SHUF, M32, RM = _lib.SCALE_E8M0_SHUFFLE, _lib.SCALE_MFMA32, _lib.SCALE_ROW_MAJOR


def both_layouts(x, xs, w, ws, dt, variant, b_layout=_lib.B_ROW_MAJOR, workspace=False):
    m, n, ks = x.shape[0], w.shape[0], xs.shape[1]
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    if b_layout == _lib.B_PRESHUFFLE:
        gw = wave_amd.b_preshuffle(gw)
    outs = []
    for layout in (SHUF, M32):
        a_s = wave_amd.scale_convert(gxs, m, ks, RM, layout)
        b_s = wave_amd.scale_convert(gws, n, ks, RM, layout)
        out = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
        wave_amd.mxfp4_gemm(gx, a_s, gw, b_s, out, a_scale_layout=layout, b_scale_layout=layout, b_layout=b_layout,
                            variant=variant, split_k=1, workspace=workspace)
        torch.cuda.synchronize()
        outs.append(out.float().cpu().numpy())
    return outs


def check(x, xs, w, ws, dt, shuf, m32, what):
    m = x.shape[0]
    rows = np.unique(np.concatenate([np.arange(0, m, 37), np.arange(255, m, 256), [m - 1]]))
    assert_close(shuf[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), dt, what + ": rows vs oracle")
    assert np.array_equal(shuf, m32, equal_nan=True), what + ": e8m0_shuffle and MFMA32 scales give different bits"


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("variant,m,n,k", [
    (_lib.VARIANT_T256x256_W4x2, 4100, 4096, 1024),   # 272 tiles of 256x256, ragged M: the last tile row runs past M
    (_lib.VARIANT_T256x192_W4x2, 4352, 3072, 1024),   # 272 tiles of 256x192
    (_lib.VARIANT_AUTO, 4353, 4096, 768),             # the library's own choice, the shortest K the kernel takes
])
def test_persistent_kernel_reads_shuffled_scales_in_place(variant, m, n, k, dt):
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=100, scale_hi=154)
    shuf, m32 = both_layouts(x, xs, w, ws, dt, variant)
    check(x, xs, w, ws, dt, shuf, m32, f"{m}x{n}x{k}")


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_bdirect_kernel_reads_shuffled_scales_in_place(dt):
    m, n, k = 4400, 4096, 2048  # 288 tiles; preshuffled B: AUTO and the variant by name take the B-direct kernel
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=5, scale_lo=110, scale_hi=140)
    for variant in (_lib.VARIANT_T256x256_W1x4_BDIRECT, _lib.VARIANT_AUTO):
        shuf, m32 = both_layouts(x, xs, w, ws, dt, variant, b_layout=_lib.B_PRESHUFFLE)
        check(x, xs, w, ws, dt, shuf, m32, f"B-direct, variant {variant}")


def test_with_scratch_the_library_re_lays_shuffled_scales_and_gives_the_same_bits():
    """With a workspace the call converts the shuffled scales to MFMA32 order first (one 5 us launch costs less than
    the kernel's doubled scale requests) and may cut a sparse last round along K (288 tiles on 256 CUs); without
    one it reads them in place.  Same bits either way where the summation order is the same (no cut: K = 1024)."""
    m, n, k = 4608, 4096, 8192
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=12, scale_lo=120, scale_hi=134)
    shuf, m32 = both_layouts(x, xs, w, ws, torch.bfloat16, _lib.VARIANT_T256x256_W4x2, workspace=None)
    check(x, xs, w, ws, torch.bfloat16, shuf, m32, "scratch: re-laid, last round cut")
    x, xs, w, ws = orc.make_inputs(4100, 4096, 1024, seed=13, scale_lo=120, scale_hi=134)
    with_ws, _ = both_layouts(x, xs, w, ws, torch.float32, _lib.VARIANT_T256x256_W4x2, workspace=None)
    without, _ = both_layouts(x, xs, w, ws, torch.float32, _lib.VARIANT_T256x256_W4x2, workspace=False)
    assert np.array_equal(with_ws, without)


def test_nan_and_extreme_scales_stay_in_their_rows_and_columns():
    """Scale byte 255 (NaN) in one group of one row of A and one row of B, bytes 0 and 200 elsewhere: the NaN
    poisons exactly that row and that column of C."""
    m, n, k = 4100, 4096, 1024
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=3, scale_lo=124, scale_hi=130)
    xs[1234, 7], ws[2345, 30] = 255, 255
    xs[17, 0], ws[4095, 31] = 0, 200
    shuf, m32 = both_layouts(x, xs, w, ws, torch.float32, _lib.VARIANT_T256x256_W4x2)
    nan = np.isnan(shuf)
    want = np.zeros_like(nan)
    want[1234, :] = True
    want[:, 2345] = True
    assert np.array_equal(nan, want)
    check(x, xs, w, ws, torch.float32, shuf, m32, "NaN / extreme scales")
