"""Pins of the CPU oracle (no GPU).  The reference stores no vectors for the
MXFP4 GEMM path, so each oracle function is checked against something the
mathematics fixes and that a plausible mistake would break: closed forms,
IEEE bit patterns, exact-rational brute force, an independent second
statement (numpy reshape/permute vs C index formulas vs a torch port), and
the layouts' defining "lane l reads base + c*l" properties."""

import glob
import os
from fractions import Fraction

import numpy as np
import pytest

from oracle import c_oracle
from oracle import mxfp4_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))


# ---------------------------------------------------------------- decode ----
def e2m1_closed_form(code: int) -> Fraction:
    """OCP MX e2m1: sign bit, 2 exponent bits (bias 1), 1 mantissa bit."""
    s, e, m = (code >> 3) & 1, (code >> 1) & 3, code & 1
    mag = Fraction(m, 2) if e == 0 else Fraction(2) ** (e - 1) * (1 + Fraction(m, 2))
    return -mag if s else mag


def test_e2m1_table_matches_closed_form():
    for code in range(16):
        assert Fraction(float(orc.E2M1_LUT[code])) == e2m1_closed_form(code)
        assert int(orc.E2M1_TWICE[code]) == 2 * e2m1_closed_form(code)
    # code 8 is negative zero, not positive zero
    assert orc.E2M1_LUT[8:9].view(np.uint32)[0] == 0x80000000
    assert orc.E2M1_LUT[0:1].view(np.uint32)[0] == 0


def test_nibble_order_low_first():
    # byte 0x21: low nibble 1 (0.5) is element 0, high nibble 2 (1.0) element 1
    out = orc.mxfp4_to_f32(np.array([[0x21, 0xF7]], dtype=np.uint8))
    assert out.tolist() == [[0.5, 1.0, 6.0, -6.0]]
    assert c_oracle.mxfp4_to_f32(np.array([[0x21, 0xF7]], dtype=np.uint8)).tolist() == [[0.5, 1.0, 6.0, -6.0]]


def test_e8m0_bit_patterns():
    s = np.arange(256, dtype=np.uint8)
    for f in (orc.e8m0_to_f32, c_oracle.e8m0_to_f32):
        bits = f(s).view(np.uint32)
        assert bits[0] == 0x00400000            # 2^-127, subnormal
        for v in range(1, 255):
            assert bits[v] == v << 23           # exponent field only
        assert np.isnan(f(s)[255])
    assert orc.e8m0_to_f32(np.array([127], np.uint8))[0] == 1.0
    assert orc.e8m0_to_f32(np.array([124], np.uint8))[0] == 0.125


def test_decoders_numpy_vs_c_all_bytes():
    b = np.arange(256, dtype=np.uint8).reshape(1, 256)
    assert np.array_equal(orc.mxfp4_to_f32(b).view(np.uint32), c_oracle.mxfp4_to_f32(b).view(np.uint32))
    g = np.load(os.path.join(HERE, "golden", "g_decode_all_bytes.npz"))
    assert np.array_equal(orc.mxfp4_to_f32(g["bytes"]).view(np.uint32), g["e2m1_f32_bits"])
    assert np.array_equal(orc.e8m0_to_f32(g["bytes"].reshape(-1)).view(np.uint32), g["e8m0_f32_bits"])


def test_dequant_numpy_vs_c_bitwise():
    rng = np.random.default_rng(0)
    q = rng.integers(0, 256, size=(7, 64), dtype=np.uint8)
    s = rng.integers(0, 256, size=(7, 4), dtype=np.uint8)
    a, b = orc.dequant_f32(q, s), c_oracle.dequant_f32(q, s)
    assert np.array_equal(np.isnan(a), np.isnan(b))
    m = ~np.isnan(a)
    assert np.array_equal(a.view(np.uint32)[m], b.view(np.uint32)[m])


# --------------------------------------------------------------- layouts ----
@pytest.mark.parametrize("m,ks", [(256, 64), (32, 8), (4093, 224), (96, 13), (1, 1)])
def test_e8m0_shuffle_three_statements_agree(m, ks):
    rng = np.random.default_rng(m * 1000 + ks)
    scale = rng.integers(0, 256, size=(m, ks), dtype=np.uint8)
    permuted = orc.e8m0_shuffle_padded(scale)           # reshape/permute
    indexed = c_oracle.e8m0_shuffle_padded(scale)       # flat index formula, C
    assert np.array_equal(permuted, indexed)
    sn = (ks + 7) // 8 * 8
    r, k = np.meshgrid(np.arange(m), np.arange(ks), indexing="ij")
    flat = orc.e8m0_shuffle_flat_index(r, k, sn)        # flat index formula, numpy
    assert np.array_equal(permuted.reshape(-1)[flat], scale)
    # bijection on the padded buffer
    sm = (m + 255) // 256 * 256
    rr, kk = np.meshgrid(np.arange(sm), np.arange(sn), indexing="ij")
    allflat = orc.e8m0_shuffle_flat_index(rr, kk, sn).reshape(-1)
    assert np.array_equal(np.sort(allflat), np.arange(sm * sn))
    # inverse
    assert np.array_equal(orc.e8m0_unshuffle(permuted, m, ks), scale)


def test_e8m0_shuffle_lane_dword_property():
    """Inside one 256-byte tile, lane l (row l%16, K group l/16 of a 128-wide
    K step) finds, in the dword at tile + 4*l, byte [kh*2 + rh] = the scale of
    row l%16 + 16*rh and group kh*4 + l/16."""
    rng = np.random.default_rng(5)
    scale = rng.integers(0, 256, size=(64, 16), dtype=np.uint8)
    buf = orc.e8m0_shuffle_padded(scale).reshape(-1)
    ksp = 16
    for rt in range(2):
        for kt in range(2):
            tile = rt * (ksp // 8) * 256 + kt * 256
            for lane in range(64):
                for kh in range(2):
                    for rh in range(2):
                        got = buf[tile + 4 * lane + kh * 2 + rh]
                        want = scale[rt * 32 + rh * 16 + lane % 16, kt * 8 + kh * 4 + lane // 16]
                        assert got == want


def test_e8m0_shuffle_reference_slice_is_lossless_when_aligned():
    rng = np.random.default_rng(6)
    scale = rng.integers(0, 256, size=(256, 32), dtype=np.uint8)
    assert np.array_equal(orc.e8m0_shuffle(scale), orc.e8m0_shuffle_padded(scale))
    # and it is a permutation of the input bytes
    assert np.array_equal(np.sort(orc.e8m0_shuffle(scale).reshape(-1)), np.sort(scale.reshape(-1)))


def test_mfma32_scale_layout_is_a_bijection_with_the_lane_property():
    """Own layout: per (row tile, K tile) block, lane (g%2)*32 + r%32 reads one
    dword whose byte t is the scale of group 2t + g%2."""
    rng = np.random.default_rng(11)
    m, ks = 70, 19
    scale = rng.integers(1, 256, size=(m, ks), dtype=np.uint8)
    buf = orc.mfma32_scale_layout(scale)
    sm, sn = 96, 24
    assert buf.shape == (sm, sn)
    rr, gg = np.meshgrid(np.arange(sm), np.arange(sn), indexing="ij")
    allflat = orc.mfma32_scale_flat_index(rr, gg, sn // 8).reshape(-1)
    assert np.array_equal(np.sort(allflat), np.arange(sm * sn))
    flat = buf.reshape(-1)
    for rt in range(3):
        for kt in range(3):
            for lane in range(64):
                for t in range(4):
                    r, g = rt * 32 + lane % 32, kt * 8 + 2 * t + lane // 32
                    want = scale[r, g] if r < m and g < ks else 0
                    assert flat[(rt * 3 + kt) * 256 + lane * 4 + t] == want


@pytest.mark.parametrize("n,kp", [(16, 32), (64, 128), (48, 96)])
def test_b_preshuffle_statements_agree(n, kp):
    rng = np.random.default_rng(n + kp)
    b = rng.integers(0, 256, size=(n, kp), dtype=np.uint8)
    permuted = orc.b_preshuffle(b)
    assert np.array_equal(permuted, c_oracle.b_preshuffle(b))
    r, k = np.meshgrid(np.arange(n), np.arange(kp), indexing="ij")
    assert np.array_equal(permuted.reshape(-1)[orc.b_preshuffle_flat_index(r, k, kp)], b)
    assert np.array_equal(np.sort(permuted.reshape(-1)), np.sort(b.reshape(-1)))


def test_b_preshuffle_lane_16_bytes_property():
    """For the 16x128 MFMA operand (16 rows, 64 packed bytes) lane l (row l%16,
    K chunk l/16) finds its 16 bytes at tile + 16*l."""
    rng = np.random.default_rng(7)
    n, kp = 32, 128
    b = rng.integers(0, 256, size=(n, kp), dtype=np.uint8)
    flat = orc.b_preshuffle(b).reshape(-1)
    for nb in range(n // 16):
        for kstep in range(kp // 64):
            tile = nb * 16 * kp + kstep * 1024
            for lane in range(64):
                got = flat[tile + 16 * lane: tile + 16 * lane + 16]
                row, chunk = nb * 16 + lane % 16, kstep * 4 + lane // 16
                assert np.array_equal(got, b[row, chunk * 16: chunk * 16 + 16])


# ------------------------------------------------------------------ GEMM ----
def brute_force_exact(x, xs, w_t, ws):
    """Textbook sum over k with exact rationals."""
    m, kp = x.shape
    n = w_t.shape[0]
    k = kp * 2
    a = orc.unpack_nibbles(x)
    b = orc.unpack_nibbles(w_t)
    out = [[Fraction(0)] * n for _ in range(m)]
    for i in range(m):
        for j in range(n):
            acc = Fraction(0)
            for e in range(k):
                va = e2m1_closed_form(int(a[i, e])) * Fraction(2) ** (int(xs[i, e // 32]) - 127)
                vb = e2m1_closed_form(int(b[j, e])) * Fraction(2) ** (int(ws[j, e // 32]) - 127)
                acc += va * vb
            out[i][j] = acc
    return out


@pytest.mark.parametrize("seed,lo,hi", [(0, 124, 130), (1, 100, 154), (2, 90, 110)])
def test_gemm_oracles_vs_exact_rationals(seed, lo, hi):
    m, n, k = 3, 4, 96
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed, lo, hi)
    want = brute_force_exact(x, xs, w_t, ws)
    got_np = orc.scaled_gemm_exact(x, w_t, xs, ws)
    got_c = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    for i in range(m):
        for j in range(n):
            w = float(want[i][j])
            assert got_np[i, j] == pytest.approx(w, rel=1e-14, abs=0)
            assert got_c[i, j] == pytest.approx(w, rel=1e-14, abs=0)
    # the f32 dequantise-then-matmul statements agree with it to f32 accuracy
    scale = max(abs(float(v)) for row in want for v in row)
    for f in (orc.scaled_gemm_f32, c_oracle.scaled_gemm_f32):
        got = f(x, w_t, xs, ws)
        for i in range(m):
            for j in range(n):
                assert abs(float(got[i, j]) - float(want[i][j])) <= 1e-5 * scale


def test_gemm_exactness_invariant_f32_bitwise():
    """With scales in 124..127 every product is a multiple of 2^-8 and partial
    sums stay below 2^16, so any summation order gives the same f32: the f32
    oracles must then equal the exact oracle bit for bit."""
    x, xs, w_t, ws = orc.make_inputs(16, 24, 512, 3, 124, 127)
    exact = orc.scaled_gemm_exact(x, w_t, xs, ws)
    assert np.array_equal(exact.astype(np.float32).astype(np.float64), exact)
    assert np.array_equal(orc.scaled_gemm_f32(x, w_t, xs, ws), exact.astype(np.float32))
    assert np.array_equal(c_oracle.scaled_gemm_f32(x, w_t, xs, ws), exact.astype(np.float32))


def test_gemm_torch_port_agrees():
    torch = pytest.importorskip("torch")
    from oracle import torch_oracle

    x, xs, w_t, ws = orc.make_inputs(32, 48, 256, 4, 124, 127)
    got = torch_oracle.torch_scaled_gemm_mxfp4(torch.from_numpy(x), torch.from_numpy(w_t),
                                               torch.from_numpy(xs), torch.from_numpy(ws)).numpy()
    assert np.array_equal(got, orc.scaled_gemm_exact(x, w_t, xs, ws).astype(np.float32))


def test_gemm_nan_scale_poisons_row_and_column():
    x, xs, w_t, ws = orc.make_inputs(4, 5, 64, 5)
    xs[1, 0] = 255
    ws[3, 1] = 255
    for c in (orc.scaled_gemm_exact(x, w_t, xs, ws), c_oracle.scaled_gemm_exact(x, w_t, xs, ws),
              orc.scaled_gemm_f32(x, w_t, xs, ws)):
        nan = np.isnan(c)
        want = np.zeros((4, 5), bool)
        want[1, :] = True
        want[:, 3] = True
        assert np.array_equal(nan, want)


def test_gemm_rows_subset():
    x, xs, w_t, ws = orc.make_inputs(20, 8, 128, 6)
    full = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    rows = np.array([0, 7, 19])
    assert np.array_equal(c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows), full[rows])
    assert np.array_equal(orc.scaled_gemm_exact(x, w_t, xs, ws, rows=rows), full[rows])


def test_grouped_oracle_is_per_group_gemm():
    e, n, k = 3, 8, 64
    off = np.array([0, 5, 5, 9], dtype=np.int32)   # middle group empty
    x, xs, _, _ = orc.make_inputs(9, n, k, 7)
    rng = np.random.default_rng(8)
    w = rng.integers(0, 256, size=(e, n, k // 2), dtype=np.uint8)
    ws = rng.integers(124, 131, size=(e, n, k // 32), dtype=np.uint8)
    got = orc.scaled_gemm_grouped_exact(x, xs, w, ws, off)
    assert np.array_equal(got[0:5], orc.scaled_gemm_exact(x[0:5], w[0], xs[0:5], ws[0]))
    assert np.array_equal(got[5:9], orc.scaled_gemm_exact(x[5:9], w[2], xs[5:9], ws[2]))


def test_bf16_rne():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(9)
    v = np.concatenate([rng.standard_normal(4096).astype(np.float32) * 1000,
                        np.array([1.0, 1.00390625, 1.01171875, -0.0, 3.3895314e38], np.float32)])
    want = torch.from_numpy(v).to(torch.bfloat16).to(torch.float32).numpy()
    got = orc.to_bf16_rne(v)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_make_group_offsets():
    off = orc.make_group_offsets(8, 8192, 3, force_empty=(2,))
    assert off[0] == 0 and off[-1] == 8192 and off.dtype == np.int32
    assert np.all(np.diff(off) >= 0) and off[3] == off[2]


# --------------------------------------------------------------- fixtures ---
@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(HERE, "golden", "g_*x*.npz"))))
def test_golden_fixtures_match_both_oracles(path):
    g = np.load(path)
    x, xs, w_t, ws, c = g["x"], g["x_scales"], g["w_t"], g["w_scales"], g["c_exact"]
    assert np.array_equal(orc.scaled_gemm_exact(x, w_t, xs, ws), c)
    got_c = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    assert np.allclose(got_c, c, rtol=1e-14, atol=0)
    assert np.array_equal(orc.e8m0_shuffle_padded(xs), g["x_scales_shuffled"])
    assert np.array_equal(c_oracle.e8m0_shuffle_padded(ws), g["w_scales_shuffled"])
    if g["w_t_preshuffled"].size:
        assert np.array_equal(c_oracle.b_preshuffle(w_t), g["w_t_preshuffled"])


def test_flops_and_bytes_accounting():
    assert orc.gemm_flops(8192, 8192, 8192) == 2 * 8192 ** 3
    # M=16 decode shape, bf16 out
    assert orc.gemm_bytes(16, 28672, 8192, 2) == 125_767_680
    assert orc.gemm_bytes(1, 28672, 8192, 2) == 124_842_240
    assert orc.gemm_bytes(32, 28672, 8192, 2) == 126_754_816
