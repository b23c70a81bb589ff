"""Helpers shared by the GPU parity tests: move oracle inputs to the GPU, run
the operator through the C ABI, and the two comparison rules of the contract.

  f32 output : max|C - C_ref| <= 1e-3 * max|C_ref|        (the stated bound)
               and, tighter, <= F32_TIGHT * max|C_ref|     (what f32 accumulation gives)
  bf16 output: |C - C_ref| <= 2^-7 * |C_ref| + BF16_ABS * max|C_ref|
               (one bf16 ulp relative, plus the f32 accumulation noise near zero)
"""

import numpy as np
import torch

import wave_amd
from wave_amd import _lib

F32_BOUND = 1e-3
F32_TIGHT = 2e-6
BF16_REL = 2.0 ** -7
BF16_ABS = 2e-6

DEV = "cuda:0"


def to_gpu(*arrays):
    return tuple(torch.from_numpy(np.ascontiguousarray(a)).to(DEV) for a in arrays)


def run_gemm(x, xs, w_t, ws, out_dtype=torch.float32, **kw):
    """numpy uint8 operands -> numpy f32 result of wave_amd.mxfp4_gemm."""
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    m, n = x.shape[0], w_t.shape[0]
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, **kw)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def assert_f32_close(c, ref, what=""):
    ref = np.asarray(ref, dtype=np.float64)
    c = np.asarray(c, dtype=np.float64)
    assert c.shape == ref.shape, (what, c.shape, ref.shape)
    assert np.array_equal(np.isnan(c), np.isnan(ref)), f"{what}: NaN pattern differs"
    ok = ~np.isnan(ref)
    if not ok.any():
        return
    scale = np.abs(ref[ok]).max()
    err = np.abs(c[ok] - ref[ok]).max()
    assert err <= F32_BOUND * scale, f"{what}: max err {err:g} > 1e-3 * {scale:g}"
    assert err <= F32_TIGHT * scale + 1e-30, f"{what}: max err {err:g} > {F32_TIGHT:g} * {scale:g}"


def assert_bf16_close(c, ref, what=""):
    ref = np.asarray(ref, dtype=np.float64)
    c = np.asarray(c, dtype=np.float64)
    assert c.shape == ref.shape, (what, c.shape, ref.shape)
    assert np.array_equal(np.isnan(c), np.isnan(ref)), f"{what}: NaN pattern differs"
    ok = ~np.isnan(ref)
    if not ok.any():
        return
    scale = np.abs(ref[ok]).max()
    tol = BF16_REL * np.abs(ref[ok]) + BF16_ABS * scale
    bad = np.abs(c[ok] - ref[ok]) > tol
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} elements beyond one bf16 ulp"


def assert_close(c, ref, out_dtype, what=""):
    (assert_bf16_close if out_dtype == torch.bfloat16 else assert_f32_close)(c, ref, what)


TILE_VARIANTS = {
    "t256x256_w2x2": _lib.VARIANT_T256x256_W2x2,
    "t256x256_w4x2": _lib.VARIANT_T256x256_W4x2,
    "t128x128_w2x2": _lib.VARIANT_T128x128_W2x2,
    "t128x256_w2x2": _lib.VARIANT_T128x256_W2x2,
}
