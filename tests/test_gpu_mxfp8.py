"""GPU: the MXFP8 block-scaled GEMM through the C ABI against the oracle
(oracle/mxfp8_oracle.py).  Floating point: the products are exact and only the
accumulation differs.  Bound: max|C - Cref| <= 1e-3 * max|Cref| (the reference's
own test, tests/kernel/wave_gemm_mxfp_test.py:416-501, uses atol 2e-3, rtol
1e-3), and the tighter 1e-4 * max|Cref| that the hardware's fp8 dot-product
tree keeps in practice (it aligns the products of one instruction to their
largest exponent before adding, so widely spread e5m2 magnitudes and scales lose
more low bits than an f32 running sum would: 2.5e-5 measured with scales
120..134)."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import mxfp8_oracle as o8
from wave_amd import _lib

from gpu_util import DEV, assert_bf16_close, to_gpu

pytestmark = pytest.mark.gpu

def assert_f32_close(c, ref, what=""):
    ref = np.asarray(ref, dtype=np.float64)
    c = np.asarray(c, dtype=np.float64)
    assert c.shape == ref.shape and not np.isnan(c).any(), what
    scale = np.abs(ref).max()
    err = np.abs(c - ref).max()
    assert err <= 1e-3 * scale, f"{what}: max err {err:g} > 1e-3 * {scale:g}"
    assert err <= 1e-4 * scale, f"{what}: max err {err:g} > 1e-4 * {scale:g}"


VARIANTS = {"auto": _lib.VARIANT_AUTO, "t256": _lib.VARIANT_T256x256_W2x2, "t256w8": _lib.VARIANT_T256x256_W4x2,
            "t128": _lib.VARIANT_T128x128_W2x2}


def run(x, xs, w_t, ws, fmt, out_dtype=torch.float32, variant=_lib.VARIANT_AUTO):
    """With the scratch buffer (scales re-laid out first) and without (read as given): same bits."""
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    out = torch.full((x.shape[0], w_t.shape[0]), float("nan"), dtype=out_dtype, device=DEV)
    wave_amd.mxfp8_gemm(gx, gxs, gw, gws, out, elem_format=fmt, variant=variant)
    direct = torch.full_like(out, float("nan"))
    wave_amd.mxfp8_gemm(gx, gxs, gw, gws, direct, elem_format=fmt, variant=variant, workspace=False)
    torch.cuda.synchronize()
    assert torch.equal(out, direct)
    return out.float().cpu().numpy()


@pytest.mark.parametrize("fmt", [o8.E5M2, o8.E4M3], ids=["e5m2", "e4m3"])
@pytest.mark.parametrize("vname", sorted(VARIANTS))
@pytest.mark.parametrize("m,n,k", [(128, 128, 128), (256, 256, 512), (300, 200, 384), (1, 40, 256), (257, 33, 1152),
                                   (1024, 1024, 1024)])
def test_mxfp8_against_oracle(m, n, k, vname, fmt):
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + n + k, fmt=fmt, scale_lo=120, scale_hi=134)
    ref = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    assert_f32_close(run(x, xs, w_t, ws, fmt, variant=VARIANTS[vname]), ref, f"{vname} {m}x{n}x{k}")


@pytest.mark.parametrize("fmt", [(o8.E4M3, o8.E5M2), (o8.E5M2, o8.E4M3)], ids=["e4m3_x_e5m2", "e5m2_x_e4m3"])
@pytest.mark.parametrize("vname", sorted(VARIANTS))
@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (300, 200, 384), (1024, 1024, 1024)])
def test_mxfp8_mixed_formats_against_oracle(m, n, k, vname, fmt):
    """Activations and weights in different 8-bit formats (each operand of the instruction carries its own)."""
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + n + k + 1, fmt=fmt, scale_lo=120, scale_hi=134)
    ref = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    assert_f32_close(run(x, xs, w_t, ws, fmt, variant=VARIANTS[vname]), ref, f"{vname} {m}x{n}x{k}")


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fmt", [o8.E5M2, (o8.E4M3, o8.E5M2)], ids=["e5m2", "e4m3_x_e5m2"])
@pytest.mark.parametrize("m,n,k", [(4352, 4096, 512), (4100, 4352, 1024)])
def test_mxfp8_more_tiles_than_cus(m, n, k, fmt, out_dtype):
    """272 and 289 tiles of 256x256 on 256 CUs: with the scratch buffer the persistent kernel walks two tiles per
    workgroup and its request stream runs across the tile boundary; without it every tile has its own workgroup and
    the scales are read as given.  Same products in the same order: the same bits (checked in run()); rows of every
    M tile against the oracle."""
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + k, fmt=fmt, scale_lo=120, scale_hi=134)
    c = run(x, xs, w_t, ws, fmt, out_dtype=out_dtype)
    rows = np.unique(np.concatenate([np.arange(0, m, 31), [m - 1, 255, 256]]))
    ref = o8.scaled_gemm_mxfp8(x[rows], w_t, xs[rows], ws, fmt)
    if out_dtype == torch.bfloat16:
        # one bf16 ulp on top of what the f32 sums are allowed (1e-4 * max|Cref| with scales spread this wide)
        tol = 2.0 ** -7 * np.abs(ref) + 1e-4 * np.abs(ref).max()
        assert (np.abs(c[rows] - ref) <= tol).all(), f"{m}x{n}x{k}: beyond one bf16 ulp + 1e-4 * max"
    else:
        assert_f32_close(c[rows], ref, f"{m}x{n}x{k}")


@pytest.mark.parametrize("fmt_x", [o8.E5M2, o8.E4M3], ids=["e5m2", "e4m3"])
@pytest.mark.parametrize("vname", sorted(VARIANTS))
@pytest.mark.parametrize("m,n,k", [(128, 128, 128), (256, 256, 512), (300, 200, 384), (1, 40, 256), (257, 33, 1152),
                                   (1024, 1024, 1024)])
def test_mxfp8_activations_against_mxfp4_weights(m, n, k, vname, fmt_x):
    """8-bit A against packed e2m1 B [N, K/2] (the mixed operand types of the scaled MMA,
    wave_lang/kernel/wave/constraints.py:425-431; the reference holds no test of them)."""
    fmt = (fmt_x, o8.E2M1)
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + n + k + 2, fmt=fmt, scale_lo=120, scale_hi=134)
    ref = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    assert_f32_close(run(x, xs, w_t, ws, fmt, variant=VARIANTS[vname]), ref, f"{vname} {m}x{n}x{k}")


@pytest.mark.parametrize("fmt_w", [o8.E5M2, o8.E4M3], ids=["e5m2", "e4m3"])
@pytest.mark.parametrize("vname", sorted(VARIANTS))
@pytest.mark.parametrize("m,n,k", [(128, 128, 128), (256, 256, 512), (300, 200, 384), (1, 40, 256), (257, 33, 1152),
                                   (1024, 1024, 1024)])
def test_mxfp4_activations_against_mxfp8_weights(m, n, k, vname, fmt_w):
    """Packed e2m1 A [M, K/2] against 8-bit B: the other order of the mixed operand types
    (wave_lang/kernel/wave/constraints.py:425-431; the reference holds no test of either)."""
    fmt = (o8.E2M1, fmt_w)
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + n + k + 5, fmt=fmt, scale_lo=120, scale_hi=134)
    assert x.shape == (m, k // 2) and w_t.shape == (n, k)
    ref = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    assert_f32_close(run(x, xs, w_t, ws, fmt, variant=VARIANTS[vname]), ref, f"{vname} {m}x{n}x{k}")


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_mxfp4_against_mxfp8_one_hot_and_more_tiles_than_cus(out_dtype):
    """One-hot rows of B (1.0 at one position, scale 1) read back columns of dequantised A exactly (every e2m1
    value times a power of two is a bf16 number), on 272 tiles: the persistent kernel with the scratch buffer."""
    m, n, k = 4352, 4096, 512
    fmt = (o8.E2M1, o8.E5M2)
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=4, fmt=fmt, scale_lo=118, scale_hi=136)
    w_t[:] = 0
    ws[:] = 127
    one = int(np.nonzero(o8.E5M2_TABLE == 1.0)[0][0])
    pos = (np.arange(n) * 37) % k
    w_t[np.arange(n), pos] = one
    c = run(x, xs, w_t, ws, fmt, out_dtype=out_dtype)
    from oracle import mxfp4_oracle as o4
    a = o4.mxfp4_to_f32(x).astype(np.float64) * o4.e8m0_to_f32(xs).astype(np.float64).repeat(32, axis=1)
    assert np.array_equal(c, a[:, pos].astype(np.float32))


def test_both_operands_e2m1_is_refused():
    x, xs, w_t, ws = o8.make_inputs_mxfp8(64, 64, 256, seed=1, fmt=(o8.E2M1, o8.E2M1))
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    out = torch.empty(64, 64, dtype=torch.float32, device=DEV)
    with pytest.raises(ValueError):
        wave_amd.mxfp8_gemm(gx, gxs, gw, gws, out, elem_format=(o8.E2M1, o8.E2M1))
    lib = _lib.load()
    st = lib.wave_mxfp8_gemm(gx.data_ptr(), gxs.data_ptr(), gw.data_ptr(), gws.data_ptr(), out.data_ptr(), 64, 64, 256,
                             _lib.MXFP8_E2M1, _lib.MXFP8_E2M1, 0, None, 0, 0, None)
    assert st == _lib.ERR_UNSUPPORTED


def test_mxfp8_against_mxfp4_one_hot_and_more_tiles_than_cus():
    """One-hot rows of A (1.0 at one position, scale 1) read back columns of dequantised B exactly, on 272 tiles
    (the persistent kernel with the scratch buffer, one tile per workgroup without: the same bits)."""
    m, n, k = 4352, 4096, 512
    fmt = (o8.E4M3, o8.E2M1)
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=3, fmt=fmt, scale_lo=118, scale_hi=136)
    x[:] = 0
    xs[:] = 127
    one = int(np.nonzero(o8.E4M3_TABLE == 1.0)[0][0])
    pos = (np.arange(m) * 37) % k
    x[np.arange(m), pos] = one
    c = run(x, xs, w_t, ws, fmt)
    from oracle import mxfp4_oracle as o4
    b = o4.mxfp4_to_f32(w_t).astype(np.float64) * o4.e8m0_to_f32(ws).astype(np.float64).repeat(32, axis=1)
    assert np.array_equal(c, b[:, pos].T.astype(np.float32))


def test_mxfp8_mixed_formats_from_torch_dtypes():
    """float8 tensors carry their own format: e4m3 activations against e5m2 weights, exact on one-hot rows."""
    m, n, k = 128, 96, 256
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=11, fmt=(o8.E4M3, o8.E5M2))
    x[:] = 0
    xs[:] = 127
    one = int(np.nonzero(o8.E4M3_TABLE == 1.0)[0][0])
    for r in range(m):
        x[r, (r * 7) % k] = one
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp8_gemm(gx.view(torch.float8_e4m3fn), gxs, gw.view(torch.float8_e5m2), gws, out)
    deq = o8.fp8_to_f64(w_t, o8.E5M2) * np.exp2(ws.astype(np.float64) - 127).repeat(32, axis=1)
    want = np.stack([deq[:, (r * 7) % k] for r in range(m)])
    assert np.array_equal(out.cpu().numpy().astype(np.float64), want)
    with pytest.raises(ValueError):
        wave_amd.mxfp8_gemm(gx.view(torch.float8_e4m3fn), gxs, gw, gws, out, elem_format=(o8.E5M2, o8.E5M2))


@pytest.mark.parametrize("fmt", [o8.E5M2, o8.E4M3], ids=["e5m2", "e4m3"])
def test_mxfp8_bf16_output_and_every_code(fmt):
    """Every finite byte value of the format appears in both operands."""
    m, n, k = 256, 384, 256
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=7, fmt=fmt)
    table = o8.E5M2_TABLE if fmt == o8.E5M2 else o8.E4M3_TABLE
    finite = np.nonzero(np.isfinite(table) & (np.abs(table) < 64))[0].astype(np.uint8)
    x[0, : len(finite)] = finite
    w_t[5, : len(finite)] = finite[::-1]
    ref = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    assert_f32_close(run(x, xs, w_t, ws, fmt), ref)
    assert_bf16_close(run(x, xs, w_t, ws, fmt, torch.bfloat16), ref)


def test_mxfp8_one_hot_rows_read_back_b():
    """A row of A that is 1.0 at one position picks out a column of dequantised B exactly."""
    fmt = o8.E5M2
    m, n, k = 128, 160, 256
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=3, fmt=fmt)
    x[:] = 0
    xs[:] = 127
    one = int(np.nonzero(o8.E5M2_TABLE == 1.0)[0][0])
    for r in range(m):
        x[r, (r * 5) % k] = one
    got = run(x, xs, w_t, ws, fmt)
    deq = o8.fp8_to_f64(w_t, fmt) * np.exp2(ws.astype(np.float64) - 127).repeat(32, axis=1)
    want = np.stack([deq[:, (r * 5) % k] for r in range(m)])
    assert np.array_equal(got.astype(np.float64), want)


def test_mxfp8_reference_style_and_torch_float8_inputs():
    """tests/kernel/wave_gemm_mxfp_test.py:64-91,416-501 with float8 tensors passed as they are."""
    shape = (1024, 1024, 1024)
    torch.manual_seed(5)
    x = torch.randn(shape[0], shape[2], device=DEV).to(torch.float8_e5m2)
    w_t = torch.randn(shape[1], shape[2], device=DEV).to(torch.float8_e5m2)
    x_scales = torch.randint(124, 128, (shape[0], shape[2] // 32), dtype=torch.uint8, device=DEV)
    w_scales = torch.randint(124, 128, (shape[1], shape[2] // 32), dtype=torch.uint8, device=DEV)
    out = torch.zeros(shape[0], shape[1], dtype=torch.float32, device=DEV)
    wave_amd.mxfp8_gemm(x, x_scales, w_t, w_scales, out)
    out2 = torch.zeros_like(out)
    wave_amd.mxfp8_gemm(x.view(torch.int8), x_scales, w_t.view(torch.int8), w_scales, out2)   # the reference's call
    assert torch.equal(out, out2)
    xf = x.float().cpu() * torch.exp2(x_scales.cpu().float() - 127).repeat_interleave(32, 1)
    wf = w_t.float().cpu() * torch.exp2(w_scales.cpu().float() - 127).repeat_interleave(32, 1)
    torch.testing.assert_close(torch.mm(xf, wf.T), out.cpu(), atol=2e-3, rtol=1e-3)


def test_mxfp8_argument_errors():
    lib = _lib.load()
    P = 0x1000
    g = lambda **kw: lib.wave_mxfp8_gemm(*[kw.get(k, d) for k, d in (
        ("a", P), ("as_", P), ("b", P), ("bs", P), ("c", P), ("m", 128), ("n", 128), ("k", 256), ("fmt", 1), ("fmt_b", 1), ("od", 0),
        ("ws", None), ("wsb", 0), ("variant", 0), ("stream", None))])
    assert g(k=192) == _lib.ERR_BAD_SHAPE
    assert g(m=-1) == _lib.ERR_BAD_SHAPE
    assert g(fmt=3) == _lib.ERR_BAD_ENUM
    assert g(fmt=2, fmt_b=2) == _lib.ERR_UNSUPPORTED   # (both e2m1: the MXFP4 entry point's)
    assert g(fmt_b=-1) == _lib.ERR_BAD_ENUM
    assert g(od=3) == _lib.ERR_BAD_ENUM
    assert g(variant=_lib.VARIANT_SKINNY) == _lib.ERR_UNSUPPORTED
    assert g(a=None) == _lib.ERR_NULL_POINTER
    assert g(b=P + 8) == _lib.ERR_MISALIGNED
    assert g(m=0, a=None, c=None) == _lib.OK
    with pytest.raises(ValueError):
        wave_amd.mxfp8_gemm(torch.zeros(4, 96, dtype=torch.uint8, device=DEV), torch.zeros(4, 3, dtype=torch.uint8, device=DEV),
                            torch.zeros(4, 96, dtype=torch.uint8, device=DEV), torch.zeros(4, 3, dtype=torch.uint8, device=DEV),
                            torch.zeros(4, 4, device=DEV))


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fmt", [o8.E5M2, (o8.E4M3, o8.E5M2), (o8.E5M2, o8.E2M1)], ids=["e5m2", "e4m3_x_e5m2", "e5m2_x_e2m1"])
@pytest.mark.parametrize("m,n,k", [(128, 256, 4096), (300, 500, 8192), (1024, 1024, 6400), (64, 1536, 11008)])
def test_mxfp8_few_tiles_long_k_split_by_the_library(m, n, k, fmt, out_dtype):
    """At most 128 tiles of 128x128 and a long K: with scratch the library cuts K into parts (f32 partial tiles in
    the scratch, one more launch to sum them; uneven parts for 50 and 86 K tiles), without scratch one workgroup
    walks the whole K.  Both against the oracle, and close to each other."""
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + n + k, fmt=fmt, scale_lo=120, scale_hi=134)
    ref = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    lib = _lib.load()
    assert lib.wave_mxfp8_workspace_bytes(m, n, k) > 2 * m * n * 4      # room for at least two parts
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    wave_amd.mxfp8_gemm(gx, gxs, gw, gws, out, elem_format=fmt)
    whole = torch.full_like(out, float("nan"))
    wave_amd.mxfp8_gemm(gx, gxs, gw, gws, whole, elem_format=fmt, workspace=False)
    torch.cuda.synchronize()
    for got, what in ((out, "split"), (whole, "whole K")):
        c = got.float().cpu().numpy()
        if out_dtype == torch.float32:
            assert_f32_close(c, ref, f"{what} {m}x{n}x{k}")
        else:
            # one bf16 ulp on top of what the f32 sums are allowed (1e-4 * max|Cref| with scales spread this wide)
            tol = 2.0 ** -7 * np.abs(ref) + 1e-4 * np.abs(ref).max()
            assert (np.abs(c - ref) <= tol).all(), f"{what} {m}x{n}x{k}: beyond one bf16 ulp + 1e-4 * max"
