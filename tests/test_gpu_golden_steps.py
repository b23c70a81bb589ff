"""GPU against the committed fixtures of the steps either side of the GEMM
(tests/golden/q_*.npz): independent of the input generators and of the oracle
code at test time."""

import os

import numpy as np
import pytest
import torch

import wave_amd
from wave_amd import _lib

from gpu_util import DEV

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def f32(bits):
    return torch.from_numpy(bits.view(np.float32).copy())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_quantiser_fixture(dtype):
    g = np.load(os.path.join(GOLDEN, "q_quantize_37x320.npz"))
    x = f32(g["x_f32_bits"]).to(dtype).to(DEV)          # the values are bf16-representable: exact in both types
    for layout, key in ((_lib.SCALE_ROW_MAJOR, "scales"), (_lib.SCALE_E8M0_SHUFFLE, "scales_shuffled"),
                        (_lib.SCALE_MFMA32, "scales_mfma32")):
        q, s = wave_amd.quantize_mxfp4(x, scale_layout=layout)
        assert np.array_equal(q.cpu().numpy(), g["q"])
        assert np.array_equal(s.cpu().numpy().reshape(-1), g[key].reshape(-1)[: s.numel()])


def test_moe_align_fixture():
    g = np.load(os.path.join(GOLDEN, "q_moe_align_50x3_e12_b8.npz"))
    ids = torch.from_numpy(g["topk_ids"]).to(DEV)
    sorted_ids = torch.full((len(g["sorted_ids"]),), -1, dtype=torch.int32, device=DEV)
    expert_ids = torch.full((len(g["expert_ids"]),), -1, dtype=torch.int32, device=DEV)
    total = torch.zeros(1, dtype=torch.int32, device=DEV)
    offsets = torch.zeros(13, dtype=torch.int32, device=DEV)
    wave_amd.moe_align_block_size(ids, 12, 8, sorted_ids, expert_ids, total, offsets)
    for got, key in ((sorted_ids, "sorted_ids"), (expert_ids, "expert_ids"), (total, "num_tokens_post_pad"),
                     (offsets, "expert_offsets")):
        assert np.array_equal(got.cpu().numpy(), g[key]), key


def test_silu_and_mul_fixture():
    g = np.load(os.path.join(GOLDEN, "q_silu_and_mul_9x64.npz"))
    gate, up = f32(g["gate_f32_bits"]).to(torch.bfloat16).to(DEV), f32(g["up_f32_bits"]).to(torch.bfloat16).to(DEV)
    out = wave_amd.silu_and_mul(gate, up).float().cpu().numpy().astype(np.float64)
    ref = g["out_f64"]
    assert (np.abs(out - ref) <= 2.0 ** -7 * np.abs(ref) + 1e-37).all()      # one bf16 ulp


@pytest.mark.parametrize("name,fmt", [("e5m2", _lib.MXFP8_E5M2), ("e4m3", _lib.MXFP8_E4M3)])
def test_mxfp8_fixture(name, fmt):
    g = np.load(os.path.join(GOLDEN, f"q_mxfp8_{name}_48_40_256.npz"))
    t = [torch.from_numpy(g[k]).to(DEV) for k in ("x", "x_scales", "w_t", "w_scales")]
    out = torch.empty(48, 40, dtype=torch.float32, device=DEV)
    wave_amd.mxfp8_gemm(t[0], t[1], t[2], t[3], out, elem_format=fmt)
    ref = g["c_f64"]
    err = np.abs(out.cpu().numpy().astype(np.float64) - ref).max()
    assert err <= 1e-4 * np.abs(ref).max()
