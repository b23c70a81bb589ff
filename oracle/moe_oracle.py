"""CPU oracle for the steps either side of the grouped (MoE) GEMM: token
alignment by expert and the gated activation between the two expert GEMMs.
TEST INFRASTRUCTURE ONLY: imported by the test suite; the HIP library never
calls into it.

Pins.
* ``moe_align_block_size`` restates tests/kernel/moe/torch_kernels.py:10-92 in
  numpy (integer work, bit-exact).  The reference holds no stored vectors for
  it; the test suite pins it against a plain Python loop over tokens (the
  definition: tokens of expert 0 first, in their original order, each expert's
  run padded to a multiple of the block) and against the invariants the
  definition fixes (every token exactly once, padding value elsewhere, one
  expert id per block, the padded total).
* ``silu_and_mul`` restates ``silu_and_mul_ref`` (tests/kernel/moe_test.py:
  39-40), ``gate * up / (1 + exp(-gate))``, evaluated in float64 and rounded once
  to the storage type; pinned against the closed form at 0, large positive and
  large negative gates and against ``x * sigmoid(x)`` from scipy.
"""

from __future__ import annotations

import numpy as np


def moe_align_block_size(topk_ids: np.ndarray, num_experts: int, block_size: int, sorted_len: int,
                         expert_ids_len: int):
    """topk_ids [num_tokens, top_k] (any integer type) -> (sorted_ids
    int32[sorted_len], expert_ids int32[expert_ids_len], num_tokens_post_pad
    int32[1], expert_offsets int32[num_experts+1]).

    sorted_ids holds, expert by expert, the flat indices (token * top_k + slot)
    of the entries routed to that expert in increasing order, each expert's run
    padded to a multiple of ``block_size`` with the value ``topk_ids.size``;
    entries past the padded total hold that value too
    (tests/kernel/moe/torch_kernels.py:30-35,61-92).  expert_ids[b] is the
    expert of block b for b below the padded total / block_size (:50-56; entries
    past that are left as given, here -1).  expert_offsets is the exclusive
    running sum of the padded counts (:47-51), the row offsets a grouped GEMM
    over the padded order takes; it is not an output of the reference function.
    """
    flat = np.asarray(topk_ids).reshape(-1).astype(np.int64)
    n = flat.size
    counts = np.bincount(flat, minlength=num_experts).astype(np.int64)
    blocks = (counts + block_size - 1) // block_size
    padded = blocks * block_size
    total = int(padded.sum())
    starts = np.cumsum(padded) - padded
    sorted_ids = np.full(sorted_len, n, dtype=np.int32)
    expert_ids = np.full(expert_ids_len, -1, dtype=np.int32)
    expert_ids[: total // block_size] = np.repeat(np.arange(num_experts), blocks)
    if n:
        order = np.argsort(flat * (n + 1) + np.arange(n), kind="stable")
        first = np.cumsum(counts) - counts
        local = np.arange(n) - np.repeat(first, counts)
        sorted_ids[starts[flat[order]] + local] = order
    offsets = np.zeros(num_experts + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(padded)
    return sorted_ids, expert_ids, np.array([total], dtype=np.int32), offsets


def silu_and_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """gate * up / (1 + exp(-gate)) in float64 (tests/kernel/moe_test.py:39-40)."""
    g = np.asarray(gate, dtype=np.float64)
    u = np.asarray(up, dtype=np.float64)
    with np.errstate(over="ignore"):
        return g * u / (1.0 + np.exp(-g))
