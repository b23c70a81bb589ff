"""GPU, bit-exact: the activation quantiser through the C ABI against the oracle
(oracle/quant_oracle.py), for every input type and scale layout, on ragged
shapes and special values; and, at the benchmark's full size, through properties
that need no oracle pass (the GEMM's own decoders invert it within half a step,
the tiled scale outputs are re-layouts of the row-major one)."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import mxfp4_oracle as orc
from oracle import quant_oracle as qo
from wave_amd import _lib

from gpu_util import DEV

pytestmark = pytest.mark.gpu

TORCH_DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def make_x(rows, k, seed, dtype, spread=6.0):
    """Normal values whose magnitude wanders over 2^+-spread from group to group,
    rounded to `dtype`; returned as the device tensor and its exact f32 image."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, k)) * np.exp2(rng.uniform(-spread, spread, size=(rows, k // 32)).repeat(32, axis=1))
    t = torch.from_numpy(x.astype(np.float32)).to(TORCH_DT[dtype]).to(DEV)
    return t, t.float().cpu().numpy()


def layout_of(scales_rm, layout):
    if layout == _lib.SCALE_ROW_MAJOR:
        return scales_rm
    if layout == _lib.SCALE_E8M0_SHUFFLE:
        return orc.e8m0_shuffle_padded(scales_rm)
    return orc.mfma32_scale_layout(scales_rm)


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("layout", [_lib.SCALE_ROW_MAJOR, _lib.SCALE_E8M0_SHUFFLE, _lib.SCALE_MFMA32])
@pytest.mark.parametrize("rows,k", [(1, 32), (16, 8192), (33, 96), (70, 2048 + 256), (257, 7168), (1024, 4096)])
def test_quantize_bit_exact(dtype, layout, rows, k):
    x, xf = make_x(rows, k, rows * 7 + k, dtype)
    q, s = wave_amd.quantize_mxfp4(x, scale_layout=layout)
    torch.cuda.synchronize()
    want_q, want_s = qo.quantize_mxfp4(xf)
    assert np.array_equal(q.cpu().numpy(), want_q)
    # (the oracle pads the shuffled buffer to 256 rows as the reference does, the library to 32: a prefix of it)
    assert np.array_equal(s.cpu().numpy().reshape(-1), layout_of(want_s, layout).reshape(-1)[: s.numel()])


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
def test_quantize_special_values(dtype):
    fi = torch.finfo(TORCH_DT[dtype])
    vals = [0.0, -0.0, fi.tiny, -fi.tiny, fi.tiny / 4, fi.max, -fi.max, float("inf"), float("-inf"), float("nan"),
            0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 7.0, 1.0, -1.5, 448.0, 2.0 ** -20, 3.0 * 2.0 ** -14]
    rng = np.random.default_rng(5)
    x = np.zeros((len(vals) + 4, 64), dtype=np.float32)
    for i, v in enumerate(vals):
        x[i, :32] = rng.standard_normal(32) * 0.5          # a group of ordinary values ...
        x[i, 3] = v                                        # ... with the special one among them
        x[i, 32:] = v                                      # and a group made of it alone
    x[len(vals)] = 0.0                                     # all-zero groups
    x[len(vals) + 1, :] = np.ldexp(rng.standard_normal(64), -130)   # tiny magnitudes (f32 subnormal)
    x[len(vals) + 2, :] = np.ldexp(rng.standard_normal(64), 120)    # huge (overflow to inf in f16)
    x[len(vals) + 3, :] = [4.0, 6.0] * 32
    with np.errstate(over="ignore"):
        t = torch.from_numpy(x).to(TORCH_DT[dtype]).to(DEV)
    q, s = wave_amd.quantize_mxfp4(t)
    torch.cuda.synchronize()
    want_q, want_s = qo.quantize_mxfp4(t.float().cpu().numpy())
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(q.cpu().numpy(), want_q)


def test_quantize_feeds_the_gemm_and_shuffle_flag():
    """quantise -> GEMM equals the oracle's GEMM of the oracle's quantised
    operands; shuffle=True gives e8m0_shuffle of the row-major scales."""
    a, af = make_x(48, 512, 1, "bf16", spread=2.0)
    b, bf = make_x(96, 512, 2, "bf16", spread=2.0)
    aq, asc = wave_amd.quantize_mxfp4(a, shuffle=True)
    bq, bsc = wave_amd.quantize_mxfp4(b, shuffle=True)
    out = torch.empty(48, 96, dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm(aq, asc, bq, bsc, out, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                        b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    torch.cuda.synchronize()
    oa, osa = qo.quantize_mxfp4(af)
    ob, osb = qo.quantize_mxfp4(bf)
    assert np.array_equal(asc.cpu().numpy().reshape(-1), orc.e8m0_shuffle_padded(osa).reshape(-1)[: asc.numel()])
    ref = orc.scaled_gemm_exact(oa, ob, osa, osb)
    got = out.cpu().numpy().astype(np.float64)
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max()
    # and the quantised product is the bf16 product up to the format's error: a sanity bound, not parity
    dense = af.astype(np.float64) @ bf.astype(np.float64).T
    assert np.abs(got - dense).max() <= 0.2 * np.abs(dense).max()


@pytest.mark.parametrize("layout", [_lib.SCALE_ROW_MAJOR, _lib.SCALE_E8M0_SHUFFLE, _lib.SCALE_MFMA32])
@pytest.mark.parametrize("m", [24, 100])
def test_quantize_feeds_the_decode_kernel_without_a_pass_between(m, layout):
    """A decode step: activations quantised on the device in each scale order, weights with resident scales in the
    same order, and the mid-M kernel with no scratch (so nothing can re-lay the scales out in between): the oracle's
    GEMM of the oracle's quantised operands."""
    n, k = 4096, 2048
    a, af = make_x(m, k, 3, "bf16", spread=2.0)
    b, bf = make_x(n, k, 4, "bf16", spread=2.0)
    aq, asc = wave_amd.quantize_mxfp4(a, scale_layout=layout)
    bq, bsc = wave_amd.quantize_mxfp4(b, scale_layout=layout)
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm(aq, asc, bq, bsc, out, a_scale_layout=layout, b_scale_layout=layout,
                        variant=_lib.VARIANT_MID_M, split_k=1, workspace=False)
    torch.cuda.synchronize()
    oa, osa = qo.quantize_mxfp4(af)
    ob, osb = qo.quantize_mxfp4(bf)
    cols = np.arange(0, n, 7)
    ref = orc.scaled_gemm_exact(oa, ob[cols], osa, osb[cols])
    got = out.cpu().numpy().astype(np.float64)[:, cols]
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max()


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_quantize_full_size_properties(dtype):
    """8192 x 8192 (the benchmark's activation): no oracle pass over 64M
    elements; instead (1) a strided sample of rows is bit-exact, (2) the decode
    the GEMM is specified by inverts it within half an e2m1 step everywhere,
    (3) the tiled scale outputs are re-layouts of the row-major one."""
    rows = k = 8192
    g = torch.Generator(device=DEV).manual_seed(3)
    x = (torch.randn(rows, k, device=DEV, generator=g) *
         torch.exp2(torch.randint(-8, 9, (rows, k // 32), device=DEV, generator=g).float()).repeat_interleave(32, 1)
         ).to(TORCH_DT[dtype])
    q, s = wave_amd.quantize_mxfp4(x)
    sample = slice(5, rows, 611)
    want_q, want_s = qo.quantize_mxfp4(x[sample].float().cpu().numpy())
    assert np.array_equal(q[sample].cpu().numpy(), want_q) and np.array_equal(s[sample].cpu().numpy(), want_s)
    back = wave_amd.dequant(q, s)
    step = torch.exp2(s.float() - 127).repeat_interleave(32, 1)
    xs = x.float().abs() / step
    spacing = torch.where(xs < 2, 0.5, torch.where(xs < 4, 1.0, 2.0))
    err = (back - x.float()).abs() / step
    assert bool((err <= torch.maximum(spacing / 2, xs - 6)).all())
    assert bool((xs < 7).all())                     # nothing saturates by more than the top half step
    for layout in (_lib.SCALE_E8M0_SHUFFLE, _lib.SCALE_MFMA32):
        q2, s2 = wave_amd.quantize_mxfp4(x, scale_layout=layout)
        assert torch.equal(q2, q)
        assert torch.equal(s2, wave_amd.scale_convert(s, rows, k // 32, _lib.SCALE_ROW_MAJOR, layout))


def test_quantize_argument_errors():
    lib = _lib.load()
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=DEV)
    q = torch.zeros(4, 32, dtype=torch.uint8, device=DEV)
    s = torch.zeros(4, 2, dtype=torch.uint8, device=DEV)
    call = lambda *a: lib.wave_mxfp4_quantize(*a)
    assert call(x.data_ptr(), 1, q.data_ptr(), s.data_ptr(), 4, 48, 0, None) == _lib.ERR_BAD_SHAPE
    assert call(x.data_ptr(), 3, q.data_ptr(), s.data_ptr(), 4, 64, 0, None) == _lib.ERR_BAD_ENUM
    assert call(x.data_ptr(), 1, q.data_ptr(), s.data_ptr(), 4, 64, 3, None) == _lib.ERR_BAD_ENUM
    assert call(None, 1, q.data_ptr(), s.data_ptr(), 4, 64, 0, None) == _lib.ERR_NULL_POINTER
    assert call(x.data_ptr() + 2, 1, q.data_ptr(), s.data_ptr(), 4, 64, 0, None) == _lib.ERR_MISALIGNED
    assert call(x.data_ptr(), 1, q.data_ptr(), s.data_ptr(), 0, 64, 0, None) == _lib.OK
    with pytest.raises(ValueError):
        wave_amd.quantize_mxfp4(torch.zeros(4, 48, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError):
        wave_amd.quantize_mxfp4(torch.zeros(4, 64, dtype=torch.int32, device=DEV))
