"""CPU oracle for the activation quantiser in front of the MXFP4 GEMM.
TEST INFRASTRUCTURE ONLY: imported by the test suite, the smoke check and the
CPU-baseline leg of the benchmark; the HIP library never calls into it.

What is restated.  The reference quantises activations and weights with a
third-party routine, ``aiter.get_triton_quant(aiter.QuantType.per_1x32)``
(call sites: wave_lang/kernel/wave/perf/bench_mxfp4_comparison.py:1484-1486
and :1897-1899).  aiter (github.com/ROCm/aiter) is neither vendored under the
reference nor pinned by it: the reference imports whatever checkout sits at
``/dockerx/aiter`` (bench_mxfp4_comparison.py:1470-1473).  The functions below
restate that routine's published algorithm (aiter's Triton
``_mxfp4_quant_op``: one e8m0 scale per 32 elements taken from the group's
largest magnitude rounded up at 1.75 of a binade, elements scaled by the
inverse power of two and rounded to e2m1 with round-to-nearest-even,
saturating at 6).

Pins.
* ``f32_to_e2m1_rne``  - pinned by mathematics: the test suite checks it
  against a search for the nearest e2m1 value in exact rational arithmetic
  (ties to the even code, saturation at 6) over every bf16 and f16 magnitude
  below 8 and random f32 values.
* ``mx_scale_from_amax`` - pinned against its closed form on exact powers of
  two and on both sides of the 1.75 threshold of every binade; that the
  threshold is 1.75 and the offset is -2 is taken from aiter's published
  source, which is absent here: agreement with aiter itself is **parity
  unpinned**.
* ``quantize_mxfp4``   - composition of the two; round trip through the
  reference's own decoders (``mxfp4_to_f32``/``e8m0_to_f32``,
  wave_lang/kernel/wave/utils/mxfp_utils.py:60-95) bounds the error at half
  an e2m1 step of the group's scale.  Non-finite inputs: own convention
  (stated at ``f32_to_e2m1_rne``), parity unpinned.
"""

from __future__ import annotations

import numpy as np

from .mxfp4_oracle import SCALE_GROUP_SIZE


def mx_scale_from_amax(amax: np.ndarray) -> np.ndarray:
    """Largest magnitude of a group (f32, >= 0) -> e8m0 scale byte.

    bits(amax) + 0x200000 carries into the exponent when the mantissa is at
    least 1.75; the exponent field e of the sum gives floor(log2) of the
    rounded-up magnitude, and the scale is 2^(e - 127 - 2) so that the largest
    element lands in [3.5, 7) before rounding, i.e. on 4 or 6.  Clamped
    to 2^-127 .. 2^127; zero and f32-subnormal groups get byte 0; infinities
    and NaN give byte 254.
    """
    amax = np.asarray(amax, dtype=np.float32)
    bits = amax.view(np.uint32).astype(np.int64) & 0x7FFFFFFF
    e = np.minimum((bits + 0x200000) >> 23, 255)  # a NaN with a large mantissa carries out of the field
    unbiased = np.where(e == 0, -127, np.clip(e - 127 - 2, -127, 127))
    unbiased = np.where(e == 255, 127, unbiased)
    return (unbiased + 127).astype(np.uint8)


def f32_to_e2m1_rne(q: np.ndarray) -> np.ndarray:
    """Already-scaled f32 values -> e2m1 codes 0..15 (bit 3 = sign), round to
    nearest, ties to the even code, magnitudes >= 6 (and NaN) to 6.

    Written the way the published routine does it, with float tricks rather
    than a table: below 1 the sum with 2^22 rounds to a multiple of 0.5 in
    hardware RNE; from 1 up to 6 the f32 mantissa is cut to one bit with the
    usual add-half-minus-one-plus-odd.
    """
    q = np.asarray(q, dtype=np.float32)
    bits = q.view(np.uint32)
    sign = (bits >> 28) & 0x8
    mag_bits = bits & 0x7FFFFFFF
    mag = mag_bits.view(np.float32)
    with np.errstate(invalid="ignore"):
        saturate = ~(mag < np.float32(6.0))
        small = mag < np.float32(1.0)
    magic = np.float32(2.0**22)
    with np.errstate(invalid="ignore", over="ignore"):
        sub = (mag + magic).astype(np.float32).view(np.uint32).astype(np.int64) - int(magic.view(np.uint32))
    nb = mag_bits.astype(np.int64)
    odd = (nb >> 22) & 1
    nrm = (nb + ((1 - 127) << 23) + (1 << 21) - 1 + odd) >> 22
    code = np.where(saturate, 7, np.where(small, sub, nrm))
    return (code.astype(np.uint32) | sign).astype(np.uint8)


def quantize_mxfp4(x: np.ndarray):
    """[R, K] float (f32, or bf16/f16 widened exactly to f32) -> (packed e2m1
    [R, K/2] uint8 with element 2j in the low nibble of byte j, e8m0 scales
    [R, K/32] uint8 row-major).  K must be a multiple of 32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    r, k = x.shape
    if k % SCALE_GROUP_SIZE:
        raise ValueError("K must be a multiple of 32")
    g = x.reshape(r, k // SCALE_GROUP_SIZE, SCALE_GROUP_SIZE)
    with np.errstate(invalid="ignore"):
        mag = np.abs(g)
        amax = np.where(np.isnan(mag).any(axis=-1), np.float32(np.inf), mag.max(axis=-1)).astype(np.float32)
    scale = mx_scale_from_amax(amax)
    unbiased = scale.astype(np.int32) - 127
    with np.errstate(invalid="ignore", over="ignore"):
        q = np.ldexp(g, -unbiased[..., None]).astype(np.float32)  # exact: a power-of-two factor
    codes = f32_to_e2m1_rne(q).reshape(r, k)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    return packed, scale


def quantize_bytes(rows, k, in_bytes):
    """Algorithmic traffic of one quantiser call: the input once, the packed
    elements and the scales once."""
    return rows * k * in_bytes + rows * k // 2 + rows * k // 32
