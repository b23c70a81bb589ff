"""CPU: pins of the MXFP8 oracle (oracle/mxfp8_oracle.py): the element decode
against the library routine the reference relies on (``tensor.to(float32)`` of a
float8 tensor, tests/kernel/wave_gemm_mxfp_test.py:82-83) over all byte values,
the GEMM against a brute-force loop in exact rationals."""

from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import mxfp8_oracle as o8


@pytest.mark.parametrize("fmt,dtype", [(o8.E5M2, torch.float8_e5m2), (o8.E4M3, torch.float8_e4m3fn)])
def test_decode_every_byte_equals_torch(fmt, dtype):
    b = torch.arange(256, dtype=torch.uint8)
    want = b.view(dtype).to(torch.float32).numpy().astype(np.float64)
    got = o8.fp8_to_f64(b.numpy(), fmt)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok]) and np.array_equal(np.signbit(got[ok]), np.signbit(want[ok]))


def test_known_values():
    assert o8.E5M2_TABLE[0x3C] == 1.0 and o8.E5M2_TABLE[0x7B] == 57344.0 and o8.E5M2_TABLE[0x01] == 2.0 ** -16
    assert np.isinf(o8.E5M2_TABLE[0x7C]) and np.isnan(o8.E5M2_TABLE[0x7D])
    assert o8.E4M3_TABLE[0x38] == 1.0 and o8.E4M3_TABLE[0x7E] == 448.0 and o8.E4M3_TABLE[0x01] == 2.0 ** -9
    assert np.isnan(o8.E4M3_TABLE[0x7F]) and o8.E4M3_TABLE[0x78] == 256.0     # no infinity in e4m3fn


@pytest.mark.parametrize("fmt", [o8.E5M2, o8.E4M3])
def test_gemm_equals_brute_force(fmt):
    m, n, k = 3, 4, 64
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=1, fmt=fmt, scale_lo=100, scale_hi=150)
    got = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    table = o8.E5M2_TABLE if fmt == o8.E5M2 else o8.E4M3_TABLE
    for i in range(m):
        for j in range(n):
            acc = Fraction(0)
            for kk in range(k):
                acc += (Fraction(float(table[x[i, kk]])) * Fraction(2) ** (int(xs[i, kk // 32]) - 127)
                        * Fraction(float(table[w_t[j, kk]])) * Fraction(2) ** (int(ws[j, kk // 32]) - 127))
            assert abs(Fraction(float(got[i, j])) - acc) <= abs(acc) * Fraction(1, 2 ** 45)


@pytest.mark.parametrize("fmt_x", [o8.E5M2, o8.E4M3])
def test_mixed_gemm_equals_brute_force(fmt_x):
    """8-bit activations against packed e2m1 weights: exact rationals, the nibble decoded here from its
    sign / exponent / mantissa fields (low nibble = even element), not through the oracle's table."""
    m, n, k = 3, 5, 64
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=2, fmt=(fmt_x, o8.E2M1), scale_lo=100, scale_hi=150)
    assert w_t.shape == (n, k // 2)
    got = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, (fmt_x, o8.E2M1))
    table = o8.E5M2_TABLE if fmt_x == o8.E5M2 else o8.E4M3_TABLE

    def e2m1(code):
        e, mnt = (code >> 1) & 3, code & 1
        mag = Fraction(mnt, 2) if e == 0 else Fraction(2) ** (e - 1) * (1 + Fraction(mnt, 2))
        return -mag if code & 8 else mag

    for i in range(m):
        for j in range(n):
            acc = Fraction(0)
            for kk in range(k):
                byte = int(w_t[j, kk // 2])
                wv = e2m1((byte >> 4) if kk & 1 else (byte & 15))
                acc += (Fraction(float(table[x[i, kk]])) * Fraction(2) ** (int(xs[i, kk // 32]) - 127)
                        * wv * Fraction(2) ** (int(ws[j, kk // 32]) - 127))
            assert abs(Fraction(float(got[i, j])) - acc) <= abs(acc) * Fraction(1, 2 ** 45) + Fraction(1, 2 ** 300)


def test_generator_rounds_to_nearest_code():
    x, xs, w_t, ws = o8.make_inputs_mxfp8(8, 8, 128, seed=0, fmt=o8.E4M3)
    assert x.dtype == np.uint8 and xs.shape == (8, 4) and np.isfinite(o8.fp8_to_f64(x, o8.E4M3)).all()
    assert ((xs >= 124) & (xs <= 127)).all()


def test_b8_preshuffle_is_the_stated_byte_formula_and_a_bijection():
    """Byte (r, c) of B lands at ((r // 32) * (K // 128) + c // 128) * 4096 + (step * 2 + half) * 1024 +
    (32 * g + r % 32) * 16 + c % 16 with step = c % 128 // 64, half = c % 64 // 32, g = c % 32 // 16: the formula
    of include/wave_mxfp4.h, byte by byte, against the reshape / transpose statement."""
    for n, k in [(32, 128), (96, 384), (64, 1024)]:
        b = np.arange(n * k, dtype=np.int64).reshape(n, k)      # every byte its own label
        got = o8.b8_preshuffle(b).reshape(-1)
        assert sorted(got.tolist()) == list(range(n * k))
        r, c = np.divmod(np.arange(n * k), k)
        cc = c % 128
        dst = ((r // 32) * (k // 128) + c // 128) * 4096 + ((cc // 64) * 2 + (cc % 64) // 32) * 1024 \
            + (32 * ((cc % 32) // 16) + r % 32) * 16 + c % 16
        want = np.empty(n * k, dtype=np.int64)
        want[dst] = np.arange(n * k)
        assert np.array_equal(got, want), (n, k)
    # a lane's two 16-byte halves of a K step are 32 bytes apart in K, 1024 bytes apart in the block
    b = np.arange(32 * 128, dtype=np.int64).reshape(32, 128)
    p = o8.b8_preshuffle(b).reshape(-1)
    lane, step = 37, 1   # g = 1, row 5
    lo = p[(step * 2 + 0) * 1024 + lane * 16:][:16]
    hi = p[(step * 2 + 1) * 1024 + lane * 16:][:16]
    assert np.array_equal(lo, b[5, 64 + 16:64 + 32]) and np.array_equal(hi, b[5, 64 + 48:64 + 64])
    with pytest.raises(ValueError):
        o8.b8_preshuffle(np.zeros((48, 128), dtype=np.uint8))
