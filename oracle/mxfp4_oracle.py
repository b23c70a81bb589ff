"""CPU oracle for the MXFP4 block-scaled GEMM path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the arithmetic the reference defines in
``wave_lang/kernel/wave/utils/mxfp_utils.py`` (input generator, e2m1 unpack,
e8m0 decode, the two host-side layout shuffles and the dequantise-then-matmul
GEMM).  Nothing here is shipped or measured as the product: only the test
suite, the smoke check and the CPU-baseline leg of the benchmark may import
it.  The HIP library never calls into it.

How each function is pinned (the reference holds no stored vectors for this
path, so the pins are mathematical):

* ``mxfp4_to_f32``      - OCP MX e2m1 closed form (sign, 2-bit exponent,
                          1-bit mantissa) and hand-written byte examples.
* ``e8m0_to_f32``       - IEEE-754 bit patterns (``s << 23``), ``ldexp``.
* ``e8m0_shuffle``      - three statements that must agree: reshape/permute,
                          the flat index formula, a bijection check; plus the
                          "lane l reads the dword at tile + 4*l" property.
* ``b_preshuffle``      - reshape/permute vs the byte offset formula; plus
                          the "lane l reads 16 B at tile + 16*l" property.
* ``scaled_gemm_f32``   - brute force with exact rationals on tiny shapes and
                          the block-exact integer oracle below.
* ``scaled_gemm_exact`` - exact rationals on tiny shapes.
  Bitwise agreement of the f32 sum with the reference's ``torch.mm`` is
  parity unpinned by design: the summation order of an f32 GEMM is not part
  of the contract, so GEMM results are compared within a stated tolerance.
"""

from __future__ import annotations

import numpy as np

# Hardware scale group size of the MX formats
# (wave_lang/kernel/wave/utils/mxfp_utils.py:17).
SCALE_GROUP_SIZE = 32

# e2m1 code -> value; bit 3 is the sign, so code 8 is -0.0
# (wave_lang/kernel/wave/utils/mxfp_utils.py:65-82).
E2M1_LUT = np.array(
    [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
     -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
    dtype=np.float32,
)

# Twice the e2m1 value as an integer (every e2m1 value is a multiple of 0.5).
E2M1_TWICE = np.array(
    [0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], dtype=np.int32
)


# --------------------------------------------------------------------------
# element decode
# --------------------------------------------------------------------------
def unpack_nibbles(packed: np.ndarray) -> np.ndarray:
    """[R, K/2] uint8 -> [R, K] uint8 codes; element 2j is the LOW nibble of
    byte j, element 2j+1 the HIGH nibble
    (wave_lang/kernel/wave/utils/mxfp_utils.py:62-64)."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = packed & 0xF
    out[..., 1::2] = packed >> 4
    return out


def mxfp4_to_f32(packed: np.ndarray) -> np.ndarray:
    """Packed e2m1 -> f32 through the 16-entry table
    (wave_lang/kernel/wave/utils/mxfp_utils.py:60-83)."""
    return E2M1_LUT[unpack_nibbles(packed)]


def e8m0_to_f32(s: np.ndarray) -> np.ndarray:
    """e8m0 byte -> f32 ``2^(s-127)``; 255 -> NaN; 0 -> 2^-127 (an f32
    subnormal, bits 0x00400000)
    (wave_lang/kernel/wave/utils/mxfp_utils.py:86-95)."""
    s = np.asarray(s, dtype=np.uint8)
    with np.errstate(over="ignore"):
        out = np.ldexp(np.float32(1.0), s.astype(np.int32) - 127).astype(np.float32)
    out[s == 255] = np.float32("nan")
    return out


def dequant_f32(packed: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """[R, K/2] codes x [R, K/32] scales -> [R, K] f32: each value times the
    scale of its 32-element group
    (wave_lang/kernel/wave/utils/mxfp_utils.py:135-143)."""
    v = mxfp4_to_f32(packed)
    s = e8m0_to_f32(np.repeat(np.asarray(scales, dtype=np.uint8),
                              SCALE_GROUP_SIZE, axis=-1))
    with np.errstate(over="ignore", invalid="ignore"):
        return v * s


# --------------------------------------------------------------------------
# GEMM
# --------------------------------------------------------------------------
def scaled_gemm_f32(x, w_t, x_scales, w_scales) -> np.ndarray:
    """The reference GEMM: dequantise both operands to f32 and multiply in
    f32, ``C = deq(x) @ deq(w_t).T`` with ``w_t`` stored ``[N, K/2]``
    (wave_lang/kernel/wave/utils/mxfp_utils.py:131-143; the reference takes
    the transposed view ``[K/2, N]`` and undoes it at :136)."""
    a = dequant_f32(x, x_scales)
    b = dequant_f32(w_t, w_scales)
    return a @ b.T


def scaled_gemm_exact(x, w_t, x_scales, w_scales, rows=None) -> np.ndarray:
    """Block-exact GEMM in f64.  Per 32-element group the dot product of
    ``2a * 2b`` is an exact integer (|.| <= 32*144); it is scaled by
    ``2^(sa+sb-256)`` (exact in f64 unless it underflows past 2^-1074) and the
    K/32 group terms are added in f64.  Scale byte 255 poisons the element
    with NaN as the reference does.  ``rows`` optionally restricts the result
    to a subset of M rows (for sampling big problems)."""
    x = np.asarray(x, dtype=np.uint8)
    w_t = np.asarray(w_t, dtype=np.uint8)
    xs = np.asarray(x_scales, dtype=np.uint8)
    ws = np.asarray(w_scales, dtype=np.uint8)
    if rows is not None:
        x, xs = x[rows], xs[rows]
    m, kp = x.shape
    n = w_t.shape[0]
    g = (kp * 2) // SCALE_GROUP_SIZE
    a = E2M1_TWICE[unpack_nibbles(x)].astype(np.float32).reshape(m, g, 32)
    b = E2M1_TWICE[unpack_nibbles(w_t)].astype(np.float32).reshape(n, g, 32)
    out = np.zeros((m, n), dtype=np.float64)
    for j in range(g):
        # integer-valued f32 products; |sum| <= 4608 < 2^24 so f32 is exact
        d = (a[:, j, :] @ b[:, j, :].T).astype(np.float64)
        e = (xs[:, j].astype(np.int64)[:, None] +
             ws[:, j].astype(np.int64)[None, :] - 256)
        out += np.ldexp(d, e)
    nan_rows = (xs == 255).any(axis=1)
    nan_cols = (ws == 255).any(axis=1)
    if nan_rows.any() or nan_cols.any():
        out[nan_rows, :] = np.nan
        out[:, nan_cols] = np.nan
    return out


def scaled_gemm_grouped_exact(x, x_scales, w_t, w_scales, offsets) -> np.ndarray:
    """Grouped (MoE) GEMM: rows ``offsets[e]:offsets[e+1]`` of ``x`` use
    expert ``e``'s ``w_t[e]`` ``[N, K/2]`` and ``w_scales[e]``.  The reference
    has no grouped MXFP4 kernel; this is its GEMM oracle applied per group
    (the per-expert loop of tests/kernel/moe_test.py:175-246)."""
    offsets = np.asarray(offsets, dtype=np.int64)
    n = w_t.shape[1]
    out = np.zeros((x.shape[0], n), dtype=np.float64)
    for e in range(len(offsets) - 1):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            out[lo:hi] = scaled_gemm_exact(x[lo:hi], w_t[e], x_scales[lo:hi],
                                           w_scales[e])
    return out


# --------------------------------------------------------------------------
# host-side layouts (input formats of the drop-in API)
# --------------------------------------------------------------------------
def e8m0_shuffle_padded(scale: np.ndarray) -> np.ndarray:
    """Scale matrix [m, n] -> tile-ordered buffer of the PADDED shape
    (ceil(m/256)*256, ceil(n/8)*8): view(sm/32, 2, 16, sn/8, 2, 4)
    .permute(0, 3, 5, 2, 4, 1)
    (wave_lang/kernel/wave/utils/mxfp_utils.py:121-127)."""
    scale = np.asarray(scale, dtype=np.uint8)
    m, n = scale.shape
    sm = (m + 255) // 256 * 256
    sn = (n + 7) // 8 * 8
    padded = np.zeros((sm, sn), dtype=np.uint8)
    padded[:m, :n] = scale
    t = padded.reshape(sm // 32, 2, 16, sn // 8, 2, 4)
    t = np.ascontiguousarray(t.transpose(0, 3, 5, 2, 4, 1))
    return t.reshape(sm, sn)


def e8m0_shuffle(scale: np.ndarray) -> np.ndarray:
    """Reference behaviour including the final slice back to [m, n]
    (wave_lang/kernel/wave/utils/mxfp_utils.py:128).  The slice drops bytes of
    valid rows when m is not a multiple of 32 or n not a multiple of 8; the
    reference only uses it where neither happens."""
    m, n = np.asarray(scale).shape
    return np.ascontiguousarray(e8m0_shuffle_padded(scale)[:m, :n])


def e8m0_shuffle_flat_index(r, k, ks_padded):
    """Flat byte offset of scale (row r, group k) in the shuffled buffer whose
    padded row length is ``ks_padded``
    (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:520-527)."""
    r = np.asarray(r, dtype=np.int64)
    k = np.asarray(k, dtype=np.int64)
    return ((r // 32) * ((ks_padded // 8) * 256) + (k // 8) * 256 +
            ((k % 8) % 4) * 64 + ((r % 32) % 16) * 4 +
            ((k % 8) // 4) * 2 + (r % 32) // 16)


def e8m0_unshuffle(shuffled: np.ndarray, m: int, n: int) -> np.ndarray:
    """Inverse of ``e8m0_shuffle_padded`` restricted to the logical [m, n]
    (coordinate form of
    examples/python/mxfp4_scale_preshuffle_visualize.py:176-212)."""
    flat = np.asarray(shuffled, dtype=np.uint8).reshape(-1)
    sn = (n + 7) // 8 * 8
    r, k = np.meshgrid(np.arange(m), np.arange(n), indexing="ij")
    return flat[e8m0_shuffle_flat_index(r, k, sn)]


def mfma32_scale_flat_index(r, g, k_tiles):
    """Flat byte offset of scale (row r, group g) in the library's own MFMA32
    order (no counterpart in the reference): per 32-row tile and K tile of 8
    groups a 256-byte block; the lane (g%2)*32 + r%32 of the 32x32x64 scaled MFMA
    holds, in byte (g%8)//2, the scale of (r, g)."""
    r = np.asarray(r, dtype=np.int64)
    g = np.asarray(g, dtype=np.int64)
    return ((r // 32) * k_tiles + g // 8) * 256 + ((g % 2) * 32 + r % 32) * 4 + (g % 8) // 2


def mfma32_scale_layout(scale: np.ndarray) -> np.ndarray:
    """Scale matrix [m, n] -> MFMA32-ordered buffer of ceil(m/32)*32 x
    ceil(n/8)*8 bytes, padding 0."""
    scale = np.asarray(scale, dtype=np.uint8)
    m, n = scale.shape
    sm, sn = (m + 31) // 32 * 32, (n + 7) // 8 * 8
    out = np.zeros(sm * sn, dtype=np.uint8)
    r, g = np.meshgrid(np.arange(m), np.arange(n), indexing="ij")
    out[mfma32_scale_flat_index(r, g, sn // 8)] = scale
    return out.reshape(sm, sn)


def b_preshuffle(b: np.ndarray) -> np.ndarray:
    """[N, K/2] packed weights -> same shape, each 16-row x 32-byte tile
    reordered from [n, k_sub, k_elem] to [k_sub, n, k_elem]:
    view(N/16, 16, Kp/32, 2, 16).permute(0, 2, 3, 1, 4)
    (wave_lang/kernel/wave/utils/mxfp_utils.py:98-110)."""
    b = np.asarray(b, dtype=np.uint8)
    n, kp = b.shape
    t = b.reshape(n // 16, 16, kp // 32, 2, 16)
    return np.ascontiguousarray(t.transpose(0, 2, 3, 1, 4)).reshape(n, kp)


def b_preshuffle_flat_index(n, kb, kp):
    """Flat byte offset of packed byte (row n, byte kb) after ``b_preshuffle``
    (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:472-483)."""
    n = np.asarray(n, dtype=np.int64)
    kb = np.asarray(kb, dtype=np.int64)
    within = (kb // 32) * 512 + ((kb // 16) % 2) * 256 + (n % 16) * 16 + kb % 16
    return (n // 16) * 16 * kp + within


# --------------------------------------------------------------------------
# seeded inputs
# --------------------------------------------------------------------------
def make_inputs(m, n, k, seed, scale_lo=124, scale_hi=130, a_scale_range=None):
    """Seeded synthetic operands: nibbles uniform 0..15, scales uniform in
    [scale_lo, scale_hi] inclusive.  Returns (x [m,k/2], x_scales [m,k/32],
    w_t [n,k/2], w_scales [n,k/32]), all uint8.  Shape and distributions
    follow wave_lang/kernel/wave/utils/mxfp_utils.py:20-57; the random stream
    is numpy's PCG64, not torch's."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    w_t = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    lo, hi = a_scale_range if a_scale_range is not None else (scale_lo, scale_hi)
    xs = rng.integers(lo, hi + 1, size=(m, k // 32), dtype=np.uint8)
    ws = rng.integers(scale_lo, scale_hi + 1, size=(n, k // 32), dtype=np.uint8)
    return x, xs, w_t, ws


def make_group_offsets(num_experts, total_rows, seed, force_empty=()):
    """Ragged group sizes: ``total_rows`` rows dealt multinomially over
    ``num_experts`` groups; groups listed in ``force_empty`` get zero rows.
    Returns int32 offsets of length num_experts+1."""
    rng = np.random.default_rng(seed)
    p = np.ones(num_experts)
    for e in force_empty:
        p[e] = 0.0
    p /= p.sum()
    counts = rng.multinomial(total_rows, p)
    off = np.zeros(num_experts + 1, dtype=np.int32)
    off[1:] = np.cumsum(counts)
    return off


def to_bf16_rne(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 (round to nearest even) returned as f32 values; the
    reference's bf16 output is ``arith.truncf`` of the f32 accumulator
    (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:120-122)."""
    x = np.asarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    out = rounded.astype(np.uint32).view(np.float32)
    return np.where(np.isnan(x), x, out)


def gemm_flops(m, n, k):
    """2*M*N*K (wave_lang/kernel/wave/perf/benchmark_mxfp4.py:78-79)."""
    return 2 * m * n * k


def gemm_bytes(m, n, k, out_bytes):
    """Algorithmic traffic of one GEMM
    (wave_lang/kernel/wave/perf/benchmark_mxfp4.py:82-85)."""
    return m * k // 2 + m * k // 32 + n * k // 2 + n * k // 32 + m * n * out_bytes
