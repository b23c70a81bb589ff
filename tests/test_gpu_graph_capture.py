"""The library's launches under HIP graph capture: every entry point takes its scratch from the caller and
enqueues kernels only (no allocation, no memset node, no synchronisation), so a captured sequence replays with the
eager results, bit for bit, also with eager work of the program between the replays."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, to_gpu

pytestmark = pytest.mark.gpu


def test_captured_gemm_sequence_replays_with_eager_results():
    # (the last three: the mid-M kernel's 32-row block on one round of strips, with two workgroups per CU, and its
    # 128-row block)
    shapes = [(1024, 1024, 8192), (16, 4096, 4096), (512, 768, 16384), (300, 200, 1248), (2304, 2304, 1024),
              (32, 16384, 2048), (24, 36864, 1024), (100, 12288, 1024)]
    ops = []
    for i, (m, n, k) in enumerate(shapes):
        x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=40 + i, scale_lo=120, scale_hi=134)
        ops.append(to_gpu(x, xs, w_t, ws) + (torch.empty(m, n, dtype=torch.bfloat16 if i % 2 else torch.float32, device=DEV),))
    act = torch.randn(512, 4096, device=DEV, dtype=torch.bfloat16)

    def sequence():
        for gx, gxs, gw, gws, out in ops:
            wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out)
        return wave_amd.quantize_mxfp4(act, scale_layout=_lib.SCALE_MFMA32)

    q_eager, s_eager = sequence()  # also sizes the cached scratch buffers, so nothing is allocated under capture
    torch.cuda.synchronize()
    eager = [o[4].clone() for o in ops]

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        sequence()  # warm-up on the capture stream
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            q_graph, s_graph = sequence()
    torch.cuda.current_stream().wait_stream(stream)
    for replay in range(3):
        for o in ops:
            o[4].fill_(float("nan"))
        q_graph.zero_()
        s_graph.zero_()
        # eager work of the program between the replays, on the same scratch
        wave_amd.mxfp4_gemm(*ops[(replay + 1) % len(ops)][:4], torch.empty_like(ops[(replay + 1) % len(ops)][4]))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for want, o in zip(eager, ops):
            assert torch.equal(want, o[4]), f"replay {replay}: {tuple(want.shape)}"
        assert torch.equal(q_graph, q_eager) and torch.equal(s_graph, s_eager)


def test_captured_grouped_sequence_replays_with_eager_results():
    """The grouped call under capture: the table-driven persistent kernel (scale re-layout launch that also builds
    the M tile table; a sparsely filled last round cut along K and summed by a second launch, decided on the device)
    and the serving-batch path (one launch of the mid-M kernel)."""
    cases = []
    for i, (e, n, k, rows) in enumerate([(4, 2048, 8192, 9300), (6, 4096, 1024, 3000), (8, 4096, 2048, 64)]):
        off = orc.make_group_offsets(e, rows, seed=70 + i)
        x, xs, _, _ = orc.make_inputs(rows, 1, k, 70 + i, scale_lo=122, scale_hi=132)
        rng = np.random.default_rng(170 + i)
        w = rng.integers(0, 256, size=(e, n, k // 2), dtype=np.uint8)
        ws = rng.integers(122, 133, size=(e, n, k // 32), dtype=np.uint8)
        cases.append(to_gpu(x, xs, w, ws, off) + (torch.empty(rows, n, dtype=torch.bfloat16 if i % 2 else torch.float32, device=DEV),))

    def sequence():
        for gx, gxs, gw, gws, goff, out in cases:
            wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out)

    sequence()
    torch.cuda.synchronize()
    eager = [c[5].clone() for c in cases]
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        sequence()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            sequence()
    torch.cuda.current_stream().wait_stream(stream)
    for replay in range(3):
        for c in cases:
            c[5].fill_(float("nan"))
        wave_amd.mxfp4_gemm_grouped(*cases[replay % len(cases)][:5], torch.empty_like(cases[replay % len(cases)][5]))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for want, c in zip(eager, cases):
            assert torch.equal(want, c[5]), f"replay {replay}: {tuple(want.shape)}"


def test_captured_serving_expert_mlp_and_mxfp8_b_direct_replay_with_eager_results():
    """One expert MLP at a serving batch as a captured graph (alignment, gathered quantiser, gate/up GEMM with the
    activation and quantiser in its C write on the mid-M kernel, down GEMM), followed by an MXFP8 GEMM on a
    preshuffled B with row-major scales (its scale re-layout launch is captured too)."""
    from oracle import mxfp8_oracle as o8
    M32, RM = _lib.SCALE_MFMA32, _lib.SCALE_ROW_MAJOR
    tokens, topk, e, hidden, inter = 48, 2, 8, 1024, 1024
    g = torch.Generator(device=DEV).manual_seed(9)
    ids = torch.stack([torch.randperm(e, device=DEV, generator=g)[:topk] for _ in range(tokens)]).to(torch.int32)
    act = torch.randn(tokens, hidden, device=DEV, generator=g).to(torch.bfloat16)
    n_ent = tokens * topk

    def weights(n, k):
        w = torch.randint(0, 256, (e, n, k // 2), dtype=torch.uint8, device=DEV, generator=g)
        ws = torch.randint(121, 128, (e, n, k // 32), dtype=torch.uint8, device=DEV, generator=g)
        return w, ws

    w1, w1s = weights(2 * inter, hidden)
    w1_il = wave_amd.interleave_gate_up(w1)
    w1s_il = wave_amd.interleave_gate_up(w1s)
    w1s_il = torch.stack([wave_amd.scale_convert(w1s_il[i], 2 * inter, hidden // 32, RM, M32) for i in range(e)])
    w2, w2s = weights(hidden, inter)
    w2s = torch.stack([wave_amd.scale_convert(w2s[i], hidden, inter // 32, RM, M32) for i in range(e)])
    sorted_ids = torch.empty(n_ent, dtype=torch.int32, device=DEV)
    expert_ids = torch.empty(n_ent, dtype=torch.int32, device=DEV)
    total = torch.empty(1, dtype=torch.int32, device=DEV)
    offs = torch.empty(e + 1, dtype=torch.int32, device=DEV)
    out = torch.empty(n_ent, hidden, dtype=torch.bfloat16, device=DEV)
    x8, xs8, w8, ws8 = to_gpu(*o8.make_inputs_mxfp8(300, 512, 1024, seed=3, fmt=o8.E5M2, scale_lo=120, scale_hi=134))
    w8p = wave_amd.mxfp8_b_preshuffle(w8)
    out8 = torch.empty(300, 512, dtype=torch.float32, device=DEV)

    def sequence():
        wave_amd.moe_align_block_size(ids, e, 1, sorted_ids, expert_ids, total, offs)
        q1, s1 = wave_amd.quantize_mxfp4_rows(act, sorted_ids, topk, scale_layout=M32)
        q2, s2 = wave_amd.mxfp4_gemm_gated_quantize(q1, s1, w1_il, w1s_il, offs, a_scale_layout=M32, b_scale_layout=M32)
        wave_amd.mxfp4_gemm_grouped(q2, s2, w2, w2s, offs, out, a_scale_layout=M32, b_scale_layout=M32)
        wave_amd.mxfp8_gemm(x8, xs8, w8p, ws8, out8, elem_format=o8.E5M2, b_preshuffled=True)
        return q2, s2

    q_eager, s_eager = sequence()
    torch.cuda.synchronize()
    out_eager, out8_eager = out.clone(), out8.clone()
    assert not bool(torch.isnan(out_eager.float()).any())
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        sequence()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            q_graph, s_graph = sequence()
    torch.cuda.current_stream().wait_stream(stream)
    valid = n_ent
    for replay in range(3):
        out.fill_(float("nan"))
        out8.fill_(float("nan"))
        q_graph.zero_()
        offs.zero_()
        sorted_ids.zero_()
        wave_amd.mxfp8_gemm(x8, xs8, w8, ws8, torch.empty_like(out8), elem_format=o8.E5M2)  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, out_eager) and torch.equal(out8, out8_eager), f"replay {replay}"
        assert torch.equal(q_graph[:valid], q_eager[:valid])
