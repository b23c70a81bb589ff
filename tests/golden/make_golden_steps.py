"""Writes the golden fixtures of the steps either side of the GEMM (q_*.npz):
the activation quantiser, the MoE token alignment, the gated activation and the
MXFP8 GEMM.  The reference holds no stored vectors for them either; the data
comes from this repository's oracles (oracle/quant_oracle.py, moe_oracle.py,
mxfp8_oracle.py), which the CPU test-suite pins independently.  Data only:
inputs and expected outputs.

Run from the repository root:  python tests/golden/make_golden_steps.py
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import moe_oracle as mo  # noqa: E402
from oracle import mxfp4_oracle as orc  # noqa: E402
from oracle import mxfp8_oracle as o8  # noqa: E402
from oracle import quant_oracle as qo  # noqa: E402


def bf16_round(x):
    return orc.to_bf16_rne(np.asarray(x, dtype=np.float32))


def main():
    rng = np.random.default_rng(101)
    # quantiser: bf16-representable inputs with group magnitudes spread over 2^+-10, plus special groups
    x = rng.standard_normal((37, 320)) * np.exp2(rng.integers(-10, 11, size=(37, 10))).repeat(32, axis=1)
    x = bf16_round(x)
    x[3, :32] = 0.0
    x[4, 32:64] = bf16_round(np.float32(1.75) * np.exp2(rng.integers(-3, 4, size=32)))     # the round-up threshold
    x[5, :32] = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4                             # every rounding tie
    q, s = qo.quantize_mxfp4(x)
    np.savez_compressed(os.path.join(HERE, "q_quantize_37x320.npz"), x_f32_bits=x.view(np.uint32), q=q, scales=s,
                        scales_shuffled=orc.e8m0_shuffle_padded(s), scales_mfma32=orc.mfma32_scale_layout(s))
    print("quantize", q.shape, s.min(), s.max())

    # token alignment: 50 tokens, top-3 of 12 experts (two experts unused), block 8
    ids = np.stack([rng.permutation(10)[:3] for _ in range(50)]).astype(np.int32)
    sorted_len, eid_len = ids.size + 12 * 7, (ids.size + 12 * 7 + 7) // 8
    sorted_ids, expert_ids, total, offsets = mo.moe_align_block_size(ids, 12, 8, sorted_len, eid_len)
    np.savez_compressed(os.path.join(HERE, "q_moe_align_50x3_e12_b8.npz"), topk_ids=ids, sorted_ids=sorted_ids,
                        expert_ids=expert_ids, num_tokens_post_pad=total, expert_offsets=offsets)
    print("align", int(total[0]), offsets.tolist())

    # gated activation on bf16 inputs: the float64 value, compared within one ulp of the output type
    gate, up = bf16_round(rng.standard_normal((9, 64)) * 3), bf16_round(rng.standard_normal((9, 64)))
    np.savez_compressed(os.path.join(HERE, "q_silu_and_mul_9x64.npz"), gate_f32_bits=gate.view(np.uint32),
                        up_f32_bits=up.view(np.uint32), out_f64=mo.silu_and_mul(gate, up))

    # MXFP8, both formats
    for fmt, name in ((o8.E5M2, "e5m2"), (o8.E4M3, "e4m3")):
        a, a_s, b, b_s = o8.make_inputs_mxfp8(48, 40, 256, seed=7, fmt=fmt, scale_lo=120, scale_hi=134)
        np.savez_compressed(os.path.join(HERE, f"q_mxfp8_{name}_48_40_256.npz"), x=a, x_scales=a_s, w_t=b,
                            w_scales=b_s, c_f64=o8.scaled_gemm_mxfp8(a, b, a_s, b_s, fmt))
        print("mxfp8", name)


if __name__ == "__main__":
    main()
