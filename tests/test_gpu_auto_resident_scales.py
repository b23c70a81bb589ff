"""GPU: the library's own choice of kernel (variant 0) when both scale tensors are handed over in MFMA32 order, as a
serving stack holds them (static weights, activations straight from the quantiser).  No kernel needs a re-layout
launch then and the choice follows borders of its own: the streaming kernel for some shapes the mid-M kernel takes
with row-major scales, the 128x128 tiles between one and two rounds of strips at a short K, and, for a preshuffled
B, the B-direct mid-M kernel from 32 rows on.  One case per border, on each side of it, against the exact oracle on
the first, the last and 96 random columns of every row, and against the same call with row-major scales (same
operands, possibly another kernel: equal within the output type's tolerance)."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu
RM, M32 = _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32


def run(gx, gxs, gw, gws, m, n, dt, layout, b_layout):
    out = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, a_scale_layout=layout, b_scale_layout=layout, b_layout=b_layout)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("pre", [False, True], ids=["b_row_major", "b_preshuffled"])
@pytest.mark.parametrize("m,n,k", [
    (32, 12288, 8192),    # K = 8192 up to N = 16384: the streaming kernel up to 48 rows ...
    (49, 16384, 8192),    # ... and the mid-M kernel (preshuffled B: from 64 rows the B-direct kernel) beyond
    (64, 12288, 8192),
    (16, 40960, 4096),    # a quarter-full second round of strips: the streaming kernel up to 16 rows at K = 4096,
    (48, 40960, 8192),    # up to 64 rows at K = 8192,
    (64, 40960, 4096),    # the 128x128 tiles from 48 rows at K = 4096 (preshuffled B: the B-direct kernel from 64)
    (128, 57344, 2048),   # the same, three quarters full
    (160, 12288, 4096),   # 128 < M <= 192, K <= 4096, N <= 16384: the tiles
    (32, 20480, 4096),    # one round of strips, preshuffled B: the B-direct kernel from 32 rows
    (100, 28672, 2048),
    (256, 40960, 1024),   # above 128 rows the B-direct kernel serves one round of strips only
    (96, 8192, 4096),     # K <= 4096, preshuffled B: the B-direct kernel from N = 8192 and 48 rows on
    (48, 10240, 2048),
])
def test_library_choice_with_resident_scales(m, n, k, pre):
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + n + k, scale_lo=116, scale_hi=138)
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    b_layout = _lib.B_ROW_MAJOR
    if pre:
        gw, b_layout = wave_amd.b_preshuffle(gw), _lib.B_PRESHUFFLE
    a32 = wave_amd.scale_convert(gxs, m, k // 32, RM, M32)
    b32 = wave_amd.scale_convert(gws, n, k // 32, RM, M32)
    rng = np.random.default_rng(m + n)
    cols = np.unique(np.concatenate([[0, 1, 127, 128, n - 129, n - 128, n - 1], rng.integers(0, n, 96)]))
    ref = c_oracle.scaled_gemm_exact(x, w[cols], xs, ws[cols])
    for dt in (torch.bfloat16, torch.float32):
        got = run(gx, a32, gw, b32, m, n, dt, M32, b_layout)
        assert not np.isnan(got).any(), "unwritten elements"
        assert_close(got[:, cols], ref, dt, f"{m}x{n}x{k} resident scales, {dt}")
        # every element: the call with row-major scales (its own choice of kernel, its own summation order)
        other = run(gx, gxs, gw, gws, m, n, dt, RM, b_layout)
        scale = np.abs(other).max()
        tol = (2.0 ** -7 if dt == torch.bfloat16 else 1e-5) * scale
        assert np.abs(got - other).max() <= tol, f"{m}x{n}x{k}: resident and row-major scales disagree"
