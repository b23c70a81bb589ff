"""CPU oracle for the MXFP8 block-scaled GEMM (one byte per element, e5m2 or
e4m3, one e8m0 scale per 32 elements).  TEST INFRASTRUCTURE ONLY.

Restates ``torchScaledGemmMXFP8`` (tests/kernel/wave_gemm_mxfp_test.py:80-91):
widen the elements to f32, multiply by the scale of their group
(``e8m0_to_f32``, wave_lang/kernel/wave/utils/mxfp_utils.py:86-95), matrix
product.  The element decode, which the reference leaves to
``tensor.to(torch.float32)`` of a float8 tensor, is restated from the OCP
formats' bit fields and pinned in the test suite against that library routine
over all 256 byte values of both formats.  The product is accumulated in
float64 (every product of two scaled elements is exact there); bitwise agreement
with ``torch.mm``'s f32 summation order is parity unpinned by design, results are
compared within a tolerance.
"""

from __future__ import annotations

import numpy as np

from .mxfp4_oracle import SCALE_GROUP_SIZE, e8m0_to_f32, mxfp4_to_f32

E4M3, E5M2 = 0, 1
E2M1 = 2   # one operand of the two: packed MXFP4 [rows, K/2] against an 8-bit other (the mixed operand
           # types of the scaled MMA, wave_lang/kernel/wave/constraints.py:425-431; the reference holds no test of
           # it, the restatement is the composition of the two pinned decodes and the same f64 product)


def _decode_table(exp_bits: int, man_bits: int, bias: int, ieee_specials: bool) -> np.ndarray:
    out = np.zeros(256, dtype=np.float64)
    for b in range(256):
        sign = -1.0 if b & 0x80 else 1.0
        e = (b >> man_bits) & ((1 << exp_bits) - 1)
        m = b & ((1 << man_bits) - 1)
        if ieee_specials and e == (1 << exp_bits) - 1:          # e5m2: infinities and NaN as in IEEE
            out[b] = sign * np.inf if m == 0 else np.nan
        elif not ieee_specials and (b & 0x7F) == 0x7F:          # e4m3fn: only S.1111.111 is NaN, no infinity
            out[b] = np.nan
        elif e == 0:
            out[b] = sign * m * 2.0 ** (1 - bias - man_bits)
        else:
            out[b] = sign * (1 + m / (1 << man_bits)) * 2.0 ** (e - bias)
    return out


E4M3_TABLE = _decode_table(4, 3, 7, False)
E5M2_TABLE = _decode_table(5, 2, 15, True)


def fp8_to_f64(x: np.ndarray, fmt: int) -> np.ndarray:
    """uint8 codes -> values (float64; every fp8 value is exact in f32 too)."""
    table = E5M2_TABLE if fmt == E5M2 else E4M3_TABLE
    return table[np.asarray(x, dtype=np.uint8)]


def scaled_gemm_mxfp8(x, w_t, x_scales, w_scales, fmt) -> np.ndarray:
    """x [M, K], w_t [N, K] uint8 codes, scales [R, K/32] e8m0 -> C [M, N] float64
    (tests/kernel/wave_gemm_mxfp_test.py:80-91 with w_t = w.T).  ``fmt`` is one
    format for both operands or a pair (x format, w_t format); an E2M1 operand is
    [rows, K/2] packed, decoded by the MXFP4 oracle's table."""
    fmt_x, fmt_w = fmt if isinstance(fmt, (tuple, list)) else (fmt, fmt)
    xs = e8m0_to_f32(np.asarray(x_scales, dtype=np.uint8)).astype(np.float64).repeat(SCALE_GROUP_SIZE, axis=1)
    ws = e8m0_to_f32(np.asarray(w_scales, dtype=np.uint8)).astype(np.float64).repeat(SCALE_GROUP_SIZE, axis=1)
    def decode(codes, f):
        return mxfp4_to_f32(np.asarray(codes, dtype=np.uint8)).astype(np.float64) if f == E2M1 else fp8_to_f64(codes, f)

    return (decode(x, fmt_x) * xs) @ (decode(w_t, fmt_w) * ws).T


def make_inputs_mxfp8(m, n, k, seed, fmt, scale_lo=124, scale_hi=127):
    """Seeded operands in the manner of generate_gemm_afp8wfp8_inputs
    (tests/kernel/wave_gemm_mxfp_test.py:64-77): normal values rounded to the
    format (one for both operands, or a pair), scales uniform in
    [scale_lo, scale_hi].  Returns codes, not floats."""
    rng = np.random.default_rng(seed)
    fmt_x, fmt_w = fmt if isinstance(fmt, (tuple, list)) else (fmt, fmt)

    def quantise(v, f):
        table = E5M2_TABLE if f == E5M2 else E4M3_TABLE
        finite = np.nonzero(np.isfinite(table))[0]
        vals = table[finite]
        order = np.argsort(vals, kind="stable")
        vals, codes = vals[order], finite[order].astype(np.uint8)
        idx = np.clip(np.searchsorted(vals, v), 1, len(vals) - 1)
        lower = (v - vals[idx - 1]) <= (vals[idx] - v)
        return codes[np.where(lower, idx - 1, idx)]

    if fmt_x == E2M1:
        x = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    else:
        x = quantise(rng.standard_normal((m, k)), fmt_x)
    if fmt_w == E2M1:   # uniform nibbles, as the MXFP4 generator draws them
        w_t = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    else:
        w_t = quantise(rng.standard_normal((n, k)), fmt_w)
    xs = rng.integers(scale_lo, scale_hi + 1, size=(m, k // 32), dtype=np.uint8)
    ws = rng.integers(scale_lo, scale_hi + 1, size=(n, k // 32), dtype=np.uint8)
    return x, xs, w_t, ws


def b8_preshuffle(b: np.ndarray) -> np.ndarray:
    """The library's preshuffled order of an 8-bit B ``[N, K]`` (declared in include/wave_mxfp4.h beside
    wave_mxfp8_b_preshuffle; the reference defines ``b_preshuffle``, mxfp_utils.py:98-110, for packed MXFP4 rows
    only, so this layout has no reference counterpart and is pinned against its own byte formula in the test
    suite): blocks of 32 rows x 128 bytes, block (n // 32, kt) first by row block then by K tile, inside a block
    the 16-byte pieces as [K step][half][g][row], the piece of (step, half, g, row) holding that row's bytes
    64 * step + 32 * half + 16 * g .. + 15 of the K tile.  Same shape out, N % 32 == 0, K % 128 == 0."""
    n, k = b.shape
    if n % 32 or k % 128:
        raise ValueError("N must be a multiple of 32 and K of 128")
    t = b.reshape(n // 32, 32, k // 128, 2, 2, 2, 16)  # row block, row, K tile, step, half, g, byte
    return np.ascontiguousarray(t.transpose(0, 2, 3, 4, 5, 1, 6)).reshape(n, k)
