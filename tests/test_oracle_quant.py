"""CPU: pins of the quantiser oracle (oracle/quant_oracle.py).  The reference
holds no vectors for this step (its quantiser is a third-party routine), so the
pins are mathematical: a nearest-value search in exact rationals for the element
rounding, the closed form for the scale, and the round trip through the
reference's own decoders (restated in oracle/mxfp4_oracle.py)."""

from fractions import Fraction

import numpy as np
import pytest

from oracle import mxfp4_oracle as orc
from oracle import quant_oracle as qo

E2M1_MAGNITUDES = [Fraction(0), Fraction(1, 2), Fraction(1), Fraction(3, 2), Fraction(2), Fraction(3), Fraction(4),
                   Fraction(6)]


def nearest_code(v: float) -> int:
    """Nearest e2m1 magnitude in exact arithmetic; a tie goes to the even code;
    anything from 6 up is 6."""
    a = abs(Fraction(float(v)))
    best_d, best_c = None, None
    for c, t in enumerate(E2M1_MAGNITUDES):
        d = abs(a - t)
        if best_d is None or d < best_d or (d == best_d and c % 2 == 0):
            best_d, best_c = d, c
    return best_c | (8 if np.signbit(v) else 0)


def test_element_rounding_every_bf16_and_f16_magnitude_below_8():
    bf = (np.arange(0, 0x4100, dtype=np.uint32) << 16).view(np.float32)          # bf16: 0 .. 8.0
    hf = np.arange(0, 0x4800, dtype=np.uint16).view(np.float16).astype(np.float32)  # f16: 0 .. 8.0
    x = np.concatenate([bf, -bf, hf, -hf])
    got = qo.f32_to_e2m1_rne(x)
    want = np.array([nearest_code(v) for v in x], dtype=np.uint8)
    assert np.array_equal(got, want)


def test_element_rounding_ties_and_random_f32():
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
    # a tie goes to the even code: 0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0
    assert list(qo.f32_to_e2m1_rne(ties)) == [0, 2, 2, 4, 4, 6, 6]
    assert list(qo.f32_to_e2m1_rne(-ties)) == [8, 10, 10, 12, 12, 14, 14]
    up = np.nextafter(ties, np.float32(10))
    assert list(qo.f32_to_e2m1_rne(up)) == [1, 2, 3, 4, 5, 6, 7]
    dn = np.nextafter(ties, np.float32(0))
    assert list(qo.f32_to_e2m1_rne(dn)) == [0, 1, 2, 3, 4, 5, 6]
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(20000) * 3).astype(np.float32)
    assert np.array_equal(qo.f32_to_e2m1_rne(x), np.array([nearest_code(v) for v in x], dtype=np.uint8))
    # saturation, signed zero, non-finite
    assert list(qo.f32_to_e2m1_rne(np.array([6, 7, 1e30, np.inf, np.nan, -np.inf, 0.0, -0.0], dtype=np.float32))) == \
        [7, 7, 7, 7, 7, 15, 0, 8]


def test_scale_closed_form_every_binade():
    # amax = m * 2^E: scale exponent is E - 2 below m = 1.75 and E - 1 from there on
    for e in range(-120, 125):
        for m, bump in [(1.0, 0), (1.5, 0), (1.7499999, 0), (1.75, 1), (1.9999999, 1)]:
            amax = np.float32(np.ldexp(np.float32(m), e))
            want = e - 2 + bump + 127
            assert int(qo.mx_scale_from_amax(amax)) == want, (e, m)
    assert int(qo.mx_scale_from_amax(np.float32(0))) == 0
    assert int(qo.mx_scale_from_amax(np.float32(1e-45))) == 0           # f32 subnormal
    assert int(qo.mx_scale_from_amax(np.float32(2.0 ** -126))) == 0     # clamped at 2^-127
    assert int(qo.mx_scale_from_amax(np.float32(2.0 ** -124))) == 1
    assert int(qo.mx_scale_from_amax(np.float32(np.inf))) == 254
    assert int(qo.mx_scale_from_amax(np.float32(3.4e38))) == 254        # rounds up into the infinite binade
    for nan_bits in (0x7FC00000, 0x7FFF0000, 0x7FFFFFFF):
        assert int(qo.mx_scale_from_amax(np.array([nan_bits], dtype=np.uint32).view(np.float32))[0]) == 254


@pytest.mark.parametrize("seed,spread", [(0, 0.0), (1, 4.0), (2, 30.0)])
def test_round_trip_error_bound_and_largest_element(seed, spread):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((33, 256)) * np.exp2(rng.uniform(-spread, spread, size=(33, 8)).repeat(32, axis=1))
         ).astype(np.float32)
    q, s = qo.quantize_mxfp4(x)
    assert q.shape == (33, 128) and s.shape == (33, 8) and q.dtype == np.uint8 and s.dtype == np.uint8
    back = orc.dequant_f32(q, s).astype(np.float64)
    step = np.exp2(s.astype(np.float64) - 127).repeat(32, axis=1)      # value of one unit of the scaled element
    xs = np.abs(x.astype(np.float64)) / step
    # spacing of e2m1 at the scaled magnitude: 0.5 below 2, 1 below 4, 2 above; the error is at most half of it,
    # except above 6 (only the group's largest element can get there: up to 7 -> 6)
    spacing = np.where(xs < 2, 0.5, np.where(xs < 4, 1.0, 2.0))
    err = np.abs(back - x.astype(np.float64)) / step
    assert (err <= np.maximum(spacing / 2, xs - 6) + 1e-12).all()
    # the largest element of every group lands on 4 or 6
    top = np.abs(back).reshape(33, 8, 32).max(axis=-1) / np.exp2(s.astype(np.float64) - 127)
    assert np.isin(top, [4.0, 6.0]).all()
    # quantising what came back changes nothing when the largest element is 4 (same scale, exact values)
    q2, s2 = qo.quantize_mxfp4(back.astype(np.float32))
    same = (top == 4.0).repeat(16, axis=1)
    assert np.array_equal(s2[top == 4.0], s[top == 4.0]) and np.array_equal(q2[same], q[same])


def test_zero_group_and_shapes():
    x = np.zeros((2, 64), dtype=np.float32)
    x[1, 40] = -3.0
    q, s = qo.quantize_mxfp4(x)
    assert s[0, 0] == 0 and s[0, 1] == 0 and s[1, 0] == 0
    assert s[1, 1] == 127 - 1 + 0      # amax 3 = 1.5 * 2^1 -> exponent 1 - 2
    assert q[1, 20] == 0x0F            # element 40 (low nibble of byte 20) = -6 after division by 0.5: code 7, sign bit
    assert not q[0].any()
    with pytest.raises(ValueError):
        qo.quantize_mxfp4(np.zeros((1, 48), dtype=np.float32))


def test_committed_fixture_matches_the_oracle():
    """tests/golden/q_quantize_37x320.npz is what the oracle says today."""
    import os

    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "q_quantize_37x320.npz"))
    q, s = qo.quantize_mxfp4(g["x_f32_bits"].view(np.float32))
    assert np.array_equal(q, g["q"]) and np.array_equal(s, g["scales"])
    assert np.array_equal(orc.e8m0_shuffle_padded(s), g["scales_shuffled"])
