"""CPU: pins of the MoE glue oracle (oracle/moe_oracle.py).  The reference holds
no vectors for these steps; alignment is pinned against a plain loop over the
entries (the definition) and its invariants, the activation against closed
forms and scipy's sigmoid."""

import numpy as np
import pytest
from scipy.special import expit

from oracle import moe_oracle as mo


def align_by_loop(flat, num_experts, block_size, sorted_len, expert_ids_len):
    """The definition, one entry at a time."""
    n = len(flat)
    buckets = [[] for _ in range(num_experts)]
    for i, e in enumerate(flat):
        buckets[int(e)].append(i)
    sorted_ids, expert_ids, offsets = [], [], [0]
    for e, b in enumerate(buckets):
        pad = (-len(b)) % block_size
        sorted_ids += b + [n] * pad
        expert_ids += [e] * ((len(b) + pad) // block_size)
        offsets.append(len(sorted_ids))
    total = len(sorted_ids)
    sorted_ids += [n] * (sorted_len - total)
    expert_ids += [-1] * (expert_ids_len - len(expert_ids))
    return np.array(sorted_ids, np.int32), np.array(expert_ids, np.int32), total, np.array(offsets, np.int32)


@pytest.mark.parametrize("tokens,topk,experts,block", [(1, 2, 8, 16), (33, 2, 8, 16), (33, 2, 64, 4), (257, 4, 8, 64),
                                                       (100, 1, 3, 1), (0, 2, 4, 8)])
def test_align_equals_definition(tokens, topk, experts, block):
    rng = np.random.default_rng(tokens + experts)
    ids = rng.integers(0, experts, size=(tokens, topk))
    n = ids.size
    sorted_len = n + experts * (block - 1) + 5
    eid_len = (sorted_len + block - 1) // block
    got = mo.moe_align_block_size(ids, experts, block, sorted_len, eid_len)
    want = align_by_loop(ids.reshape(-1), experts, block, sorted_len, eid_len)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    assert int(got[2][0]) == want[2] and np.array_equal(got[3], want[3])
    # invariants: every entry exactly once, padding elsewhere, total a multiple of the block
    real = got[0][got[0] < n]
    assert np.array_equal(np.sort(real), np.arange(n)) and int(got[2][0]) % block == 0
    assert (got[0][int(got[2][0]):] == n).all()


def test_align_skewed_routing():
    ids = np.zeros((50, 2), dtype=np.int64)          # everything to expert 0 ...
    ids[7, 1] = 5                                    # ... but one entry
    s, e, total, off = mo.moe_align_block_size(ids, 8, 16, 100 + 8 * 15, 20)
    assert int(total[0]) == 112 + 16 and list(off) == [0, 112, 112, 112, 112, 112, 128, 128, 128]
    assert list(s[:99]) == [i for i in range(100) if i != 15] and (s[99:112] == 100).all()
    assert s[112] == 15 and (s[113:128] == 100).all()
    assert list(e[:8]) == [0] * 7 + [5] and (e[8:] == -1).all()


def test_silu_and_mul_closed_forms():
    g = np.array([0.0, 1.0, -1.0, 30.0, -30.0, 100.0, -100.0, 1e-4])
    u = np.array([3.0, 2.0, 2.0, 1.5, 1.5, -2.0, 7.0, 1.0])
    got = mo.silu_and_mul(g, u)
    assert got[0] == 0.0
    assert np.isclose(got[1], 2.0 / (1.0 + np.e ** -1), rtol=1e-15)
    assert np.isclose(got[2], -2.0 / (1.0 + np.e), rtol=1e-15)
    assert np.isclose(got[3], 45.0, rtol=1e-12) and abs(got[4]) < 1e-11       # x for large x, 0 for very negative x
    assert got[5] == -200.0 and got[6] == 0.0 or abs(got[6]) < 1e-40
    assert np.isclose(got[7], 1e-4 * 0.5 * (1 + 0.5e-4), rtol=1e-8)           # x/2 * (1 + x/2 + ...)
    rng = np.random.default_rng(0)
    g, u = rng.standard_normal(1000) * 4, rng.standard_normal(1000)
    assert np.allclose(mo.silu_and_mul(g, u), g * expit(g) * u, rtol=1e-13, atol=0)
