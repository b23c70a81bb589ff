"""GPU: the gate/up GEMM of a gated expert MLP with silu(gate) * up and the MXFP4 quantiser of the next GEMM's
operand fused into its C write (wave_mxfp4_gemm_gated_quantize), against the chain it replaces, bit for bit:
wave_mxfp4_gemm_grouped (bf16 out) -> wave_mxfp4_silu_and_mul_quantize on the two halves of its output, which are
themselves held to the oracles in test_gpu_configs.py / test_gpu_moe.py.  The reference's chain is
tests/kernel/moe_test.py:113-129 (GEMM, silu_and_mul, GEMM); it notes fused dynamic quantisation as not done
(wave_lang/kernel/wave/templates/test_kernels.py:74).

The weight's gate and up rows are interleaved in blocks of 32 (wave_mxfp4_interleave_gate_up, checked against numpy
here), which moves a gate element and its up element into the same lane of the MFMA result."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, to_gpu

pytestmark = pytest.mark.gpu
M32, RM = _lib.SCALE_MFMA32, _lib.SCALE_ROW_MAJOR


def np_interleave(t, block=32):
    half = t.shape[-2] // 2
    g = t[..., :half, :].reshape(*t.shape[:-2], half // block, block, t.shape[-1])
    u = t[..., half:, :].reshape(*t.shape[:-2], half // block, block, t.shape[-1])
    return np.stack([g, u], axis=-3).reshape(t.shape)


def test_interleave_gate_up_matches_numpy():
    rng = np.random.default_rng(0)
    for shape in [(128, 64), (3, 256, 36), (2, 64, 7)]:
        t = rng.integers(0, 256, size=shape, dtype=np.uint8)
        got = wave_amd.interleave_gate_up(torch.from_numpy(t).to(DEV)).cpu().numpy()
        assert np.array_equal(got, np_interleave(t)), shape


def run_chain_and_fused(counts, inter, k, seed, rows_dense=None, a_native=False):
    grouped = counts is not None
    rows = int(sum(counts)) if grouped else rows_dense
    e = len(counts) if grouped else 1
    x, xs, _, _ = orc.make_inputs(rows, 1, k, seed, scale_lo=122, scale_hi=128)
    rng = np.random.default_rng(seed + 1)
    w = rng.integers(0, 256, size=(e, 2 * inter, k // 2), dtype=np.uint8)
    ws = rng.integers(120, 127, size=(e, 2 * inter, k // 32), dtype=np.uint8)
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    n = 2 * inter
    # the chain
    c = torch.full((rows, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    if grouped:
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).to(DEV)
        wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, off, c, variant=_lib.VARIANT_T256x256_W4x2)
    else:
        off = None
        wave_amd.mxfp4_gemm(gx, gxs, gw[0], gws[0], c, variant=_lib.VARIANT_T256x256_W4x2, split_k=1)
    q_ref, s_ref = wave_amd.silu_and_mul_quantize(c[:, :inter], c[:, inter:], scale_layout=M32)
    # the fused call
    w_il, ws_il = wave_amd.interleave_gate_up(gw), wave_amd.interleave_gate_up(gws)
    a_s, kw = gxs, {}
    if a_native:
        a_s = wave_amd.scale_convert(gxs, rows, k // 32, RM, M32)
        ws_il = torch.stack([wave_amd.scale_convert(ws_il[g], n, k // 32, RM, M32) for g in range(e)])
        kw = dict(a_scale_layout=M32, b_scale_layout=M32)
    if not grouped:
        w_il, ws_il = w_il[0], ws_il[0]
    q, s = wave_amd.mxfp4_gemm_gated_quantize(gx, a_s, w_il, ws_il, off, **kw)
    torch.cuda.synchronize()
    valid = int(off[-1].item()) if grouped else rows
    assert torch.equal(q[:valid], q_ref[:valid]), "packed codes differ from the unfused chain"
    s_rm = wave_amd.scale_convert(s, rows, inter // 32, M32, RM)
    s_ref_rm = wave_amd.scale_convert(s_ref, rows, inter // 32, M32, RM)
    assert torch.equal(s_rm[:valid], s_ref_rm[:valid]), "scales differ from the unfused chain"
    # not degenerate: the activation uses most codes and several scale values
    codes = torch.bincount((q[:valid].flatten() & 15).to(torch.int64), minlength=16)
    assert int((codes > 0).sum()) >= 12 and len(torch.unique(s_rm[:valid])) >= 3
    return q, s


@pytest.mark.parametrize("a_native", [False, True])
def test_grouped_fused_matches_the_chain(a_native):
    # ragged groups, one empty, starts that are no multiples of 32; 37 x 8 = 296 tiles of 256x256 on 256 workgroups
    counts = [1000, 1033, 0, 2050, 517, 2049, 1777, 300]
    run_chain_and_fused(counts, inter=1024, k=1024, seed=41, a_native=a_native)


def test_dense_fused_matches_the_chain():
    run_chain_and_fused(None, inter=2048, k=768, seed=42, rows_dense=4400)   # 18 x 16 = 288 tiles, ragged last tile row


def test_rows_past_the_last_offset_are_left_alone_and_small_problems_are_refused():
    counts = [3000, 2000, 3500]
    rows, inter, k = 8600, 1024, 1024
    x, xs, _, _ = orc.make_inputs(rows, 1, k, 43, scale_lo=122, scale_hi=128)
    rng = np.random.default_rng(44)
    w = rng.integers(0, 256, size=(3, 2 * inter, k // 2), dtype=np.uint8)
    ws = rng.integers(120, 127, size=(3, 2 * inter, k // 32), dtype=np.uint8)
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).to(DEV)
    lib = _lib.load()
    q = torch.full((rows, inter // 2), 0xAB, dtype=torch.uint8, device=DEV)
    s = torch.full(((rows + 31) // 32 * 32, inter // 32), 0xCD, dtype=torch.uint8, device=DEV)
    ws_bytes = int(lib.wave_mxfp4_grouped_workspace_bytes(rows, 2 * inter, k, 3))
    scratch = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    w_il, ws_il = wave_amd.interleave_gate_up(gw), wave_amd.interleave_gate_up(gws)
    stream = torch.cuda.current_stream().cuda_stream
    st = lib.wave_mxfp4_gemm_gated_quantize(gx.data_ptr(), gxs.data_ptr(), w_il.data_ptr(), ws_il.data_ptr(), q.data_ptr(),
                                            s.data_ptr(), off.data_ptr(), 3, rows, 2 * inter, k, RM, RM, M32,
                                            scratch.data_ptr(), ws_bytes, stream)
    assert st == _lib.OK
    torch.cuda.synchronize()
    assert bool((q[8500:] == 0xAB).all()) and not bool((q[:8500] == 0xAB).all(dim=1).any())
    s_rm = wave_amd.scale_convert(s, rows, inter // 32, M32, RM)
    assert bool((s_rm[8500:] == 0xCD).all())
    # too few tiles for the persistent kernel, no workspace, a row-major result: refused, nothing written
    small = lib.wave_mxfp4_gemm_gated_quantize(gx.data_ptr(), gxs.data_ptr(), w_il.data_ptr(), ws_il.data_ptr(), q.data_ptr(),
                                               s.data_ptr(), off.data_ptr(), 3, 512, 2 * inter, k, RM, RM, M32,
                                               scratch.data_ptr(), ws_bytes, stream)
    assert small == _lib.ERR_UNSUPPORTED
    assert lib.wave_mxfp4_gemm_gated_quantize(gx.data_ptr(), gxs.data_ptr(), w_il.data_ptr(), ws_il.data_ptr(), q.data_ptr(),
                                              s.data_ptr(), off.data_ptr(), 3, rows, 2 * inter, k, RM, RM, M32, None, 0,
                                              stream) == _lib.ERR_UNSUPPORTED
    assert lib.wave_mxfp4_gemm_gated_quantize(gx.data_ptr(), gxs.data_ptr(), w_il.data_ptr(), ws_il.data_ptr(), q.data_ptr(),
                                              s.data_ptr(), off.data_ptr(), 3, rows, 2 * inter, k, RM, RM, RM,
                                              scratch.data_ptr(), ws_bytes, stream) == _lib.ERR_UNSUPPORTED


# ---- a small batch routed over the experts: the same epilogue in the grouped mid-M kernel ----

def run_small_batch(counts, inter, k, seed, a_native, slack_rows=0):
    """Resident weight scales (MFMA32) and a batch the grouped call gives to the mid-M kernel: far too few 256x256
    tiles for the persistent kernel, so a fused call that succeeds ran the mid-M kernel.  Against the chain through
    the same kernel (grouped GEMM, variant MID_M, bf16 out, then silu_and_mul_quantize), bit for bit."""
    e, n = len(counts), 2 * inter
    valid = int(sum(counts))
    rows = valid + slack_rows
    x, xs, _, _ = orc.make_inputs(rows, 1, k, seed, scale_lo=122, scale_hi=128)
    rng = np.random.default_rng(seed + 1)
    w = rng.integers(0, 256, size=(e, n, k // 2), dtype=np.uint8)
    ws = rng.integers(120, 127, size=(e, n, k // 32), dtype=np.uint8)
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).to(DEV)
    c = torch.full((rows, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, off, c, variant=_lib.VARIANT_MID_M)
    q_ref, s_ref = wave_amd.silu_and_mul_quantize(c[:valid, :inter], c[:valid, inter:], scale_layout=RM)
    w_il, ws_il = wave_amd.interleave_gate_up(gw), wave_amd.interleave_gate_up(gws)
    ws_il = torch.stack([wave_amd.scale_convert(ws_il[g], n, k // 32, RM, M32) for g in range(e)])
    a_s, la = gxs, RM
    if a_native:
        a_s, la = wave_amd.scale_convert(gxs, rows, k // 32, RM, M32), M32
    lib = _lib.load()
    q = torch.full((rows, inter // 2), 0xAB, dtype=torch.uint8, device=DEV)
    s = torch.full(((rows + 31) // 32 * 32, (inter // 32 + 7) // 8 * 8), 0xCD, dtype=torch.uint8, device=DEV)
    ws_bytes = int(lib.wave_mxfp4_grouped_workspace_bytes(rows, n, k, e))
    scratch = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=DEV)
    st = lib.wave_mxfp4_gemm_gated_quantize(gx.data_ptr(), a_s.data_ptr(), w_il.data_ptr(), ws_il.data_ptr(), q.data_ptr(),
                                            s.data_ptr(), off.data_ptr(), e, rows, n, k, la, M32, M32,
                                            scratch.data_ptr(), scratch.numel(), torch.cuda.current_stream().cuda_stream)
    assert st == _lib.OK, st
    torch.cuda.synchronize()
    assert torch.equal(q[:valid], q_ref), "packed codes differ from the unfused chain"
    assert bool((q[valid:] == 0xAB).all()), "rows past the last offset were written"
    s_rm = wave_amd.scale_convert(s, rows, inter // 32, M32, RM)
    assert torch.equal(s_rm[:valid], s_ref), "scales differ from the unfused chain"
    assert bool((s_rm[valid:] == 0xCD).all()), "scales of rows past the last offset were written"
    codes = torch.bincount((q[:valid].flatten() & 15).to(torch.int64), minlength=16)
    assert int((codes > 0).sum()) >= 12 and len(torch.unique(s_rm[:valid])) >= 3


@pytest.mark.parametrize("a_native", [False, True], ids=["a_scales_row_major", "a_scales_mfma32"])
@pytest.mark.parametrize("counts,inter,k", [
    ([16, 9, 0, 31, 22, 1, 40, 13], 1024, 1024),              # blocks of 32 rows (gate / up exchanged through LDS)
    ([10, 20, 5, 0, 33, 12, 7, 25], 2304, 1024),              # the same, more strips than CUs: two workgroups per CU
    ([70, 20, 64, 65, 3, 0, 50, 47], 1792, 2048),             # blocks of 64 rows, two groups of a second pass
    ([100, 0, 260, 33, 1, 150, 97, 128], 1024, 1024),         # blocks of 128 rows, a group of three passes
    ([150, 160, 140, 155, 149, 132, 141, 143], 1024, 1536),   # blocks of 192 rows
    ([250, 260, 240, 255, 249, 232, 241, 243], 2048, 1024),   # two passes of 192-row blocks (few column tiles: the
                                                              # tile kernels would leave CUs idle for whole rounds)
], ids=["bm32", "bm32_two_per_cu", "bm64", "bm128", "bm192", "bm192_two_passes"])
def test_small_batch_fused_in_the_mid_kernel_matches_the_chain(counts, inter, k, a_native):
    run_small_batch(counts, inter, k, seed=sum(counts) + k, a_native=a_native, slack_rows=37)


def _small_batch_cases(count, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        e = int(rng.integers(4, 17))
        avg = int(rng.integers(1, 140))
        counts = rng.multinomial(avg * e, rng.dirichlet(np.full(e, 2.0))).tolist()
        inter = 128 * int(rng.integers(1, 13))
        while e * (2 * inter // 128) < 128:   # experts x strips of 128 columns: at least half the CUs
            inter += 128
        out.append((i, counts, inter, 256 * int(rng.integers(4, 9)), bool(rng.integers(0, 2)), int(rng.integers(0, 40))))
    return out


@pytest.mark.parametrize("case", _small_batch_cases(10, seed=77), ids=lambda c: f"{c[0]}-E{len(c[1])}-rows{sum(c[1])}-I{c[2]}-K{c[3]}")
def test_random_small_batches_fused_in_the_mid_kernel(case):
    """Seeded expert counts dealt unevenly (Dirichlet weights: empty experts, experts of several blocks), 4 .. 16
    experts, every block height the library picks."""
    i, counts, inter, k, a_native, slack = case
    run_small_batch(counts, inter, k, seed=900 + i, a_native=a_native, slack_rows=slack)
