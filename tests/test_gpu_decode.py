"""GPU, bit-exact: element decode, dequantisation and the two layout shuffles
through the C ABI against the oracle and the golden table."""

import os

import numpy as np
import pytest
import torch

import wave_amd
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, to_gpu

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def bits(t):
    return t.cpu().numpy().view(np.uint32)


def test_e2m1_all_bytes_bit_exact():
    g = np.load(os.path.join(HERE, "golden", "g_decode_all_bytes.npz"))
    (q,) = to_gpu(g["bytes"])
    got = bits(wave_amd.mxfp4_to_f32(q))
    assert np.array_equal(got, g["e2m1_f32_bits"])
    # code 8 must come out as negative zero
    assert got[0, 2 * 8] == 0x80000000 and got[0, 2 * 0x80 + 1] == 0x80000000


def test_e8m0_all_bytes_bit_exact():
    g = np.load(os.path.join(HERE, "golden", "g_decode_all_bytes.npz"))
    (s,) = to_gpu(g["bytes"].reshape(-1))
    got = wave_amd.e8m0_to_f32(s)
    gb = bits(got)
    want = g["e8m0_f32_bits"]
    assert np.array_equal(gb[:255], want[:255])
    assert gb[0] == 0x00400000          # 2^-127 kept as a subnormal, not flushed
    assert np.isnan(got.cpu().numpy()[255])


@pytest.mark.parametrize("rows,k,seed", [(7, 64, 0), (130, 7168, 1), (1, 32, 2)])
def test_dequant_bit_exact_full_scale_range(rows, k, seed):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 256, size=(rows, k // 2), dtype=np.uint8)
    s = rng.integers(0, 256, size=(rows, k // 32), dtype=np.uint8)   # includes 0 and 255
    flat = s.reshape(-1)
    flat[0] = 0
    flat[-1] = 255 if flat.size > 1 else 0
    want = orc.dequant_f32(q, s)
    gq, gs = to_gpu(q, s)
    got = wave_amd.dequant(gq, gs).cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok])
    # same through the shuffled scale layout
    gss = wave_amd.e8m0_shuffle(gs)
    got2 = wave_amd.dequant(gq, gss, scale_layout=_lib.SCALE_E8M0_SHUFFLE).cpu().numpy()
    assert np.array_equal(got2.view(np.uint32)[ok], want.view(np.uint32)[ok])


@pytest.mark.parametrize("rows,ks", [(256, 64), (4093, 224), (33, 9), (1, 1), (6144, 224)])
def test_e8m0_shuffle_matches_oracle(rows, ks):
    rng = np.random.default_rng(rows + ks)
    s = rng.integers(0, 256, size=(rows, ks), dtype=np.uint8)
    (gs,) = to_gpu(s)
    got = wave_amd.e8m0_shuffle(gs).cpu().numpy()
    rp = (rows + 31) // 32 * 32
    assert got.shape == (rp, (ks + 7) // 8 * 8)
    assert np.array_equal(got, orc.e8m0_shuffle_padded(s)[:rp])


@pytest.mark.parametrize("rows,ks", [(256, 64), (4093, 224), (70, 264), (33, 9), (1, 1)])
def test_scale_convert_every_layout_pair(rows, ks):
    rng = np.random.default_rng(rows * 7 + ks)
    s = rng.integers(0, 256, size=(rows, ks), dtype=np.uint8)
    rp = (rows + 31) // 32 * 32
    forms = {
        _lib.SCALE_ROW_MAJOR: s,
        _lib.SCALE_E8M0_SHUFFLE: orc.e8m0_shuffle_padded(s)[:rp],
        _lib.SCALE_MFMA32: orc.mfma32_scale_layout(s),
    }
    for src, src_arr in forms.items():
        (g,) = to_gpu(src_arr)
        for dst, want in forms.items():
            got = wave_amd.scale_convert(g, rows, ks, src, dst).cpu().numpy()
            assert np.array_equal(got, want), (src, dst)
    # dequantisation reads the MFMA32 order too
    q = rng.integers(0, 256, size=(rows, ks * 16), dtype=np.uint8)
    s2 = np.clip(s, 1, 254)
    gq, gs = to_gpu(q, orc.mfma32_scale_layout(s2))
    got = wave_amd.dequant(gq, gs, scale_layout=_lib.SCALE_MFMA32).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), orc.dequant_f32(q, s2).view(np.uint32))


@pytest.mark.parametrize("n,kp", [(16, 32), (6144, 3584), (48, 96)])
def test_b_preshuffle_matches_oracle(n, kp):
    rng = np.random.default_rng(n + kp)
    b = rng.integers(0, 256, size=(n, kp), dtype=np.uint8)
    (gb,) = to_gpu(b)
    assert np.array_equal(wave_amd.b_preshuffle(gb).cpu().numpy(), orc.b_preshuffle(b))


def test_reference_named_helpers_on_gpu():
    from wave_amd.kernel.wave.utils import mxfp_utils as mu

    x, w, xs, ws = mu.generate_gemm_afp4wfp4_inputs((64, 32, 256), device=torch.device(DEV))
    assert x.is_cuda and x.shape == (64, 128) and w.shape == (128, 32)
    want = orc.mxfp4_to_f32(x.cpu().numpy())
    assert np.array_equal(mu.mxfp4_to_f32(x).cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert np.array_equal(mu.e8m0_to_f32(xs).cpu().numpy(), orc.e8m0_to_f32(xs.cpu().numpy()))
    assert np.array_equal(mu.b_preshuffle(w.T.contiguous()).cpu().numpy(),
                          orc.b_preshuffle(w.T.contiguous().cpu().numpy()))
    assert np.array_equal(mu.e8m0_shuffle(xs).cpu().numpy(), orc.e8m0_shuffle_padded(xs.cpu().numpy())[:64])
