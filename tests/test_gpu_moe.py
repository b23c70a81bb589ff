"""GPU: the steps either side of the grouped (MoE) GEMM through the C ABI.
Alignment and the gathered quantiser are integer / byte work: bit-exact against
the oracle.  The gated activation is floating point: within one unit in the last
place of the 16-bit output of the float64 oracle value (the reference's own
test allows rtol 1e-1 / atol 1e-2, tests/kernel/moe_test.py:255); the fused
activation + quantiser must equal the two separate kernels bit for bit."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import moe_oracle as mo
from oracle import mxfp4_oracle as orc
from oracle import quant_oracle as qo
from wave_amd import _lib

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def run_align(ids, experts, block, extra=3):
    n = ids.numel()
    sorted_len = n + experts * (block - 1) + extra
    eid_len = (sorted_len + block - 1) // block
    sorted_ids = torch.full((sorted_len,), -7, dtype=torch.int32, device=DEV)
    expert_ids = torch.full((eid_len,), -1, dtype=torch.int32, device=DEV)
    total = torch.full((1,), -7, dtype=torch.int32, device=DEV)
    offsets = torch.full((experts + 1,), -7, dtype=torch.int32, device=DEV)
    wave_amd.moe_align_block_size(ids, experts, block, sorted_ids, expert_ids, total, offsets)
    torch.cuda.synchronize()
    return sorted_ids.cpu().numpy(), expert_ids.cpu().numpy(), total.cpu().numpy(), offsets.cpu().numpy()


@pytest.mark.parametrize("idtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("tokens,topk,experts,block", [(1, 2, 8, 16), (33, 2, 8, 16), (33, 2, 64, 4), (4096, 2, 8, 128),
                                                       (1000, 1, 3, 1), (5000, 8, 256, 32), (70000, 2, 1024, 64),
                                                       (0, 2, 4, 8)])
def test_moe_align_bit_exact(tokens, topk, experts, block, idtype):
    rng = np.random.default_rng(tokens * 3 + experts)
    ids = rng.integers(0, experts, size=(tokens, topk))
    got = run_align(torch.from_numpy(ids).to(idtype).to(DEV), experts, block)
    n = ids.size
    want = mo.moe_align_block_size(ids, experts, block, len(got[0]), len(got[1]))
    for g, w, name in zip(got, want, ("sorted_ids", "expert_ids", "num_tokens_post_pad", "expert_offsets")):
        assert np.array_equal(g, w), name


def test_moe_align_skewed_and_empty_experts():
    ids = np.zeros((3000, 2), dtype=np.int64)     # one expert takes almost everything, most take nothing
    ids[::7, 1] = 5
    ids[11, 0] = 7
    got = run_align(torch.from_numpy(ids).to(DEV), 8, 16)
    want = mo.moe_align_block_size(ids, 8, 16, len(got[0]), len(got[1]))
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,n", [(1, 64), (33, 1024), (257, 7168), (2048, 14336)])
def test_silu_and_mul_one_ulp(dtype, rows, n):
    g = torch.Generator(device=DEV).manual_seed(rows + n)
    gate = (torch.randn(rows, n, device=DEV, generator=g) * 3).to(dtype)
    up = torch.randn(rows, n, device=DEV, generator=g).to(dtype)
    out = wave_amd.silu_and_mul(gate, up)
    torch.cuda.synchronize()
    ref = mo.silu_and_mul(gate.float().cpu().numpy(), up.float().cpu().numpy())
    got = out.float().cpu().numpy().astype(np.float64)
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)     # half the spacing relative to the binade, doubled below
    tiny = float(torch.finfo(dtype).tiny)
    assert (np.abs(got - ref) <= 2 * ulp * np.abs(ref) + tiny).all()
    # halves of one [rows, 2n] tensor, as the first expert GEMM leaves them
    both = torch.cat([gate, up], dim=1)
    out2 = wave_amd.silu_and_mul(both[:, :n], both[:, n:])
    assert torch.equal(out2, out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", [_lib.SCALE_ROW_MAJOR, _lib.SCALE_E8M0_SHUFFLE, _lib.SCALE_MFMA32])
@pytest.mark.parametrize("rows,n", [(5, 96), (300, 2048 + 512), (1024, 14336)])
def test_fused_activation_quantiser_equals_the_two_kernels(dtype, layout, rows, n):
    g = torch.Generator(device=DEV).manual_seed(rows * 3 + n)
    both = (torch.randn(rows, 2 * n, device=DEV, generator=g) * 2).to(dtype)
    gate, up = both[:, :n], both[:, n:]
    q, s = wave_amd.silu_and_mul_quantize(gate, up, scale_layout=layout)
    act = wave_amd.silu_and_mul(gate, up)
    q2, s2 = wave_amd.quantize_mxfp4(act, scale_layout=layout)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    # ... and the oracle's quantiser on the stored activation
    wq, ws = qo.quantize_mxfp4(act.float().cpu().numpy())
    assert np.array_equal(q.cpu().numpy(), wq)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gathered_quantiser_and_grouped_gemm_pipeline(dtype):
    """Routing table -> alignment (block 1: no padding) -> gathered quantiser ->
    grouped GEMM, against the oracle run expert by expert."""
    tokens, topk, experts, k, n = 300, 2, 8, 512, 256
    rng = np.random.default_rng(9)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)])
    ids[:, :][ids == 3] = 4                     # expert 3 gets nothing
    a = torch.from_numpy(rng.standard_normal((tokens, k)).astype(np.float32)).to(dtype).to(DEV)
    sorted_ids, _, total, offsets = run_align(torch.from_numpy(ids).to(DEV), experts, 1, extra=0)
    assert int(total[0]) == tokens * topk
    gq, gs = wave_amd.quantize_mxfp4_rows(a, torch.from_numpy(sorted_ids).to(DEV), topk)
    # the same rows gathered on the host and quantised by the oracle
    af = a.float().cpu().numpy()
    wq, ws = qo.quantize_mxfp4(af[sorted_ids // topk])
    assert np.array_equal(gq.cpu().numpy(), wq) and np.array_equal(gs.cpu().numpy(), ws)
    # padded order (block 16): padding rows are zero rows with zero scale bytes
    sorted_pad, _, total_pad, _ = run_align(torch.from_numpy(ids).to(DEV), experts, 16, extra=0)
    pq, ps = wave_amd.quantize_mxfp4_rows(a, torch.from_numpy(sorted_pad).to(DEV), topk)
    pad = sorted_pad >= tokens * topk
    assert pad.any() and not pq.cpu().numpy()[pad].any() and not ps.cpu().numpy()[pad].any()
    assert np.array_equal(pq.cpu().numpy()[~pad], wq) and np.array_equal(ps.cpu().numpy()[~pad], ws)
    # grouped GEMM over the sorted rows
    _, _, w_t, wsc = orc.make_inputs(1, experts * n, k, seed=2)
    w_t, wsc = w_t.reshape(experts, n, k // 2), wsc.reshape(experts, n, k // 32)
    out = torch.empty(tokens * topk, n, dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gq, gs, torch.from_numpy(w_t).to(DEV), torch.from_numpy(wsc).to(DEV),
                                torch.from_numpy(offsets).to(DEV), out)
    torch.cuda.synchronize()
    ref = orc.scaled_gemm_grouped_exact(wq, ws, w_t, wsc, offsets)
    got = out.cpu().numpy().astype(np.float64)
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max()


@pytest.mark.parametrize("size", ["serving", "prefill"])
def test_expert_mlp_chain_with_resident_scale_layouts(size):
    """One mixture-of-experts MLP (the path of tests/kernel/moe_test.py:113-246 up to its weighted sum): alignment
    -> gathered quantiser -> grouped GEMM (gate and up) -> gated activation fused into the quantiser -> grouped
    GEMM (down), every scale tensor written or kept in MFMA32 order so that no re-layout launch sits between the
    steps.  Each step against the oracle applied to the device's output of the step before: bytes exact for the
    quantisers, the GEMMs within the bf16 bound.  "serving": a few rows per expert (the mid-M kernel, one workgroup
    per expert and strip, whose blocks of rows start inside the 32-row blocks of the activations' MFMA32 scales:
    80 routed rows over 8 experts, 8 x 16 and 8 x 8 strips); "prefill": more 256x256 tiles than CUs (table-driven
    persistent kernel, groups starting at rows that are no multiples of 32), where the first GEMM with the
    activation and the quantiser fused into its C write must give the chain's q2 / s2 bit for bit."""
    tokens, topk, experts, hidden, inter = (40, 2, 8, 1024, 2048) if size == "serving" else (2600, 2, 4, 1024, 2048)
    m32 = _lib.SCALE_MFMA32
    rng = np.random.default_rng(31)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)])
    act = torch.from_numpy(rng.standard_normal((tokens, hidden)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    sorted_ids, _, total, offsets = run_align(torch.from_numpy(ids).to(DEV), experts, 1, extra=0)
    rows = tokens * topk
    assert int(total[0]) == rows and any(int(o) % 32 for o in offsets[1:-1])
    g_sorted, g_off = torch.from_numpy(sorted_ids).to(DEV), torch.from_numpy(offsets).to(DEV)

    def weights(n, k, seed):
        r = np.random.default_rng(seed)
        w = r.integers(0, 256, size=(experts, n, k // 2), dtype=np.uint8)
        ws = r.integers(118, 130, size=(experts, n, k // 32), dtype=np.uint8)
        gws = torch.stack([wave_amd.scale_convert(torch.from_numpy(ws[e]).to(DEV), n, k // 32, _lib.SCALE_ROW_MAJOR, m32)
                           for e in range(experts)])
        return w, ws, torch.from_numpy(w).to(DEV), gws

    w1, w1s, gw1, gw1s = weights(2 * inter, hidden, 1)
    w2, w2s, gw2, gw2s = weights(hidden, inter, 2)
    # gathered quantiser, scales straight into MFMA32 order
    q1, s1 = wave_amd.quantize_mxfp4_rows(act, g_sorted, topk, scale_layout=m32)
    want_q1, want_s1 = qo.quantize_mxfp4(act.float().cpu().numpy()[sorted_ids // topk])
    assert np.array_equal(q1.cpu().numpy(), want_q1)
    s1_rm = wave_amd.scale_convert(s1, rows, hidden // 32, m32, _lib.SCALE_ROW_MAJOR).cpu().numpy()
    assert np.array_equal(s1_rm, want_s1)
    # gate and up projections
    h1 = torch.full((rows, 2 * inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp4_gemm_grouped(q1, s1, gw1, gw1s, g_off, h1, a_scale_layout=m32, b_scale_layout=m32)
    torch.cuda.synchronize()
    pick = np.unique(np.concatenate([np.arange(0, rows, max(1, rows // 40)), offsets[1:-1] - 1, offsets[1:-1] % rows, [rows - 1]]))
    h1_host = h1.float().cpu().numpy()
    for e in range(experts):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        sel = pick[(pick >= lo) & (pick < hi)]
        if len(sel):
            ref = c_oracle.scaled_gemm_exact(want_q1, w1[e], want_s1, w1s[e], rows=sel)
            tol = 2.0 ** -7 * np.abs(ref).max()
            assert np.abs(h1_host[sel] - ref).max() <= tol, f"gate/up, expert {e}"
    assert not np.isnan(h1_host).any()
    # gated activation + quantiser on the device's own h1
    q2, s2 = wave_amd.silu_and_mul_quantize(h1[:, :inter], h1[:, inter:], scale_layout=m32)
    stored = wave_amd.silu_and_mul(h1[:, :inter], h1[:, inter:])
    want_q2, want_s2 = qo.quantize_mxfp4(stored.float().cpu().numpy())
    assert np.array_equal(q2.cpu().numpy(), want_q2)
    assert np.array_equal(wave_amd.scale_convert(s2, rows, inter // 32, m32, _lib.SCALE_ROW_MAJOR).cpu().numpy(), want_s2)
    if size == "prefill":
        # the same three steps as one call: interleaved gate / up weights, activation + quantiser in the C write
        w1_il = wave_amd.interleave_gate_up(gw1)
        w1s_il = torch.stack([wave_amd.scale_convert(wave_amd.interleave_gate_up(torch.from_numpy(w1s[e]).to(DEV)), 2 * inter,
                                                     hidden // 32, _lib.SCALE_ROW_MAJOR, m32) for e in range(experts)])
        fq2, fs2 = wave_amd.mxfp4_gemm_gated_quantize(q1, s1, w1_il, w1s_il, g_off, a_scale_layout=m32, b_scale_layout=m32)
        assert np.array_equal(fq2.cpu().numpy(), want_q2)
        assert np.array_equal(wave_amd.scale_convert(fs2, rows, inter // 32, m32, _lib.SCALE_ROW_MAJOR).cpu().numpy(), want_s2)
    ref_act = mo.silu_and_mul(h1_host[:, :inter], h1_host[:, inter:])
    got_act = stored.float().cpu().numpy().astype(np.float64)
    assert np.abs(got_act - ref_act).max() <= 2.0 ** -7 * max(1.0, np.abs(ref_act).max())
    # down projection
    out = torch.full((rows, hidden), float("nan"), dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp4_gemm_grouped(q2, s2, gw2, gw2s, g_off, out, a_scale_layout=m32, b_scale_layout=m32)
    torch.cuda.synchronize()
    out_host = out.float().cpu().numpy()
    for e in range(experts):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        sel = pick[(pick >= lo) & (pick < hi)]
        if len(sel):
            ref = c_oracle.scaled_gemm_exact(want_q2, w2[e], want_s2, w2s[e], rows=sel)
            assert np.abs(out_host[sel] - ref).max() <= 2.0 ** -7 * np.abs(ref).max(), f"down, expert {e}"
    assert not np.isnan(out_host).any()


def test_moe_glue_argument_errors():
    lib = _lib.load()
    P = 0x1000
    al = lib.wave_mxfp4_moe_align_block_size
    assert al(P, 0, 10, 0, 4, P, 40, P, 10, P, None, None) == _lib.ERR_BAD_SHAPE        # no experts
    assert al(P, 0, 10, 4, 0, P, 40, P, 10, P, None, None) == _lib.ERR_BAD_SHAPE        # block size 0
    assert al(P, 0, 10, 4, 4, P, 5, P, 10, P, None, None) == _lib.ERR_BAD_SHAPE         # sorted_ids too short
    assert al(P, 0, 10, 2000, 4, P, 40, P, 10, P, None, None) == _lib.ERR_UNSUPPORTED
    assert al(None, 0, 10, 4, 4, P, 40, P, 10, P, None, None) == _lib.ERR_NULL_POINTER
    assert al(P, 2, 10, 4, 4, P, 40, P, 10, P, None, None) == _lib.ERR_BAD_ENUM
    assert al(P + 4, 1, 10, 4, 4, P, 40, P, 10, P, None, None) == _lib.ERR_MISALIGNED
    sm = lib.wave_mxfp4_silu_and_mul
    assert sm(P, P, P, 64, 64, 64, 0, 4, 64, None) == _lib.ERR_BAD_ENUM                 # f32 is not taken
    assert sm(P, P, P, 64, 64, 64, 1, 4, 60, None) == _lib.ERR_BAD_SHAPE
    assert sm(P, P, P, 32, 64, 64, 1, 4, 64, None) == _lib.ERR_BAD_SHAPE                # stride below n
    assert sm(P, None, P, 64, 64, 64, 1, 4, 64, None) == _lib.ERR_NULL_POINTER
    assert sm(P, P + 8, P, 64, 64, 64, 1, 4, 64, None) == _lib.ERR_MISALIGNED
    sq = lib.wave_mxfp4_silu_and_mul_quantize
    assert sq(P, P, 64, 64, 1, P, P, 4, 40, 0, None) == _lib.ERR_BAD_SHAPE              # n % 32
    assert sq(P, P, 64, 64, 1, P, P, 4, 64, 3, None) == _lib.ERR_BAD_ENUM
    qr = lib.wave_mxfp4_quantize_rows
    assert qr(P, 1, 4, None, 1, P, P, 4, 64, 0, None) == _lib.ERR_NULL_POINTER
    assert qr(P, 1, 4, P, 0, P, P, 4, 64, 0, None) == _lib.ERR_BAD_SHAPE
    with pytest.raises(ValueError):
        wave_amd.silu_and_mul(torch.zeros(4, 64, device=DEV), torch.zeros(4, 64, device=DEV))   # f32
