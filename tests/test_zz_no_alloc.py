"""GPU: wave_mxfp4_gemm_static, the entry point that allocates nothing (its scratch is a fixed array inside the
library's device image), through the C ABI against wave_mxfp4_gemm with a caller-provided workspace: the same
kernels in the same order, so the same bits.  Two calls in a row share the array, the second on a smaller
problem, so stale contents of the first must not leak into the second."""

import numpy as np
import pytest
import torch

from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu


def both(lib, m, n, k, out_dtype, seed, split_k=0, variant=0, asl=0, bsl=0):
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=seed, scale_lo=120, scale_hi=134)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    od = _lib.OUT_BF16 if out_dtype == torch.bfloat16 else _lib.OUT_F32
    stream = torch.cuda.current_stream().cuda_stream
    got = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    st = lib.wave_mxfp4_gemm_static(gx.data_ptr(), gxs.data_ptr(), gw.data_ptr(), gws.data_ptr(), got.data_ptr(),
                                    m, n, k, od, asl, bsl, 0, split_k, variant, stream)
    assert st == _lib.OK, (st, lib.wave_mxfp4_last_hip_error())
    # (the library's own split takes the parts that fit: the same scratch size for the same parts and bits)
    need = min(lib.wave_mxfp4_workspace_bytes(m, n, k, split_k, variant), lib.wave_mxfp4_static_scratch_bytes())
    ws_buf = torch.empty(max(need, 256), dtype=torch.uint8, device=DEV)
    want = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    st = lib.wave_mxfp4_gemm(gx.data_ptr(), gxs.data_ptr(), gw.data_ptr(), gws.data_ptr(), want.data_ptr(),
                             m, n, k, od, asl, bsl, 0, split_k, ws_buf.data_ptr(), need, variant, stream)
    assert st == _lib.OK
    torch.cuda.synchronize()
    return got, want, (x, xs, w_t, ws)


@pytest.mark.parametrize("first,second", [
    # (m, n, k, out dtype, split_k): a K split by the library itself (f32 parts in the scratch), then a smaller one
    ((1024, 1024, 8192, torch.bfloat16, 0), (512, 768, 2048, torch.bfloat16, 0)),
    # re-laid scales of a many-tile problem, then an explicit split of a small one
    ((2304, 2048, 1024, torch.float32, 1), (200, 136, 1024, torch.float32, 4)),
    # a decode shape whose K is split over workgroups, then a plain one
    ((16, 2048, 16384, torch.bfloat16, 0), (16, 512, 1024, torch.bfloat16, 0)),
])
def test_static_scratch_matches_workspace_entry_point(first, second):
    lib = _lib.load()
    assert lib.wave_mxfp4_static_scratch_bytes() == 16 << 20
    for i, (m, n, k, dt, split) in enumerate((first, second)):
        got, want, (x, xs, w_t, ws) = both(lib, m, n, k, dt, seed=70 + i, split_k=split)
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), (m, n, k)
        assert_close(got.float().cpu().numpy(), orc.scaled_gemm_exact(x, w_t, xs, ws), dt, f"{m}x{n}x{k} vs oracle")


def test_static_scratch_rejects_what_does_not_fit():
    lib = _lib.load()
    p = 0x1000
    # 8 splits of 8192 x 8192 f32 parts: 2 GiB of partial sums
    assert lib.wave_mxfp4_workspace_bytes(8192, 8192, 8192, 8, 0) > lib.wave_mxfp4_static_scratch_bytes()
    st = lib.wave_mxfp4_gemm_static(p, p, p, p, p, 8192, 8192, 8192, 1, 0, 0, 0, 8, 0, None)
    assert st == _lib.ERR_WORKSPACE
    assert b"static" in lib.wave_mxfp4_last_hip_error()
    # the headline shape fits
    assert lib.wave_mxfp4_workspace_bytes(8192, 8192, 8192, 0, 0) <= lib.wave_mxfp4_static_scratch_bytes()
    # argument errors come before the size test
    assert lib.wave_mxfp4_gemm_static(None, p, p, p, p, 64, 64, 256, 0, 0, 0, 0, 1, 0, None) == _lib.ERR_NULL_POINTER
    assert lib.wave_mxfp4_gemm_static(p, p, p, p, p, 64, 64, 48, 0, 0, 0, 0, 1, 0, None) == _lib.ERR_BAD_SHAPE


def test_static_entry_allocates_nothing_and_replays_from_a_captured_graph():
    """After the set-up call (wave_mxfp4_static_scratch_bytes, which looks the array's address up) and one call per
    kernel (which loads it), calls leave the device's free memory where it was; a call captured into a HIP graph
    replays with the eager bits, with eager calls on the same array between the replays; and a problem of 16384^3
    whose scales are already in MFMA32 order is not refused for the scratch other layouts of that shape would need."""
    lib = _lib.load()
    assert lib.wave_mxfp4_static_scratch_bytes() == 16 << 20
    m, n, k = 2304, 2048, 1024   # re-laid scales in the scratch, the persistent kernel
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=91, scale_lo=120, scale_hi=134)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    small = torch.empty(64, 256, dtype=torch.float32, device=DEV)

    def call(stream, dst=out):
        st = lib.wave_mxfp4_gemm_static(gx.data_ptr(), gxs.data_ptr(), gw.data_ptr(), gws.data_ptr(), dst.data_ptr(),
                                        dst.shape[0], dst.shape[1], k, _lib.OUT_BF16 if dst.dtype == torch.bfloat16 else _lib.OUT_F32,
                                        0, 0, 0, 0, 0, stream)
        assert st == _lib.OK, (st, lib.wave_mxfp4_last_hip_error())

    cur = torch.cuda.current_stream().cuda_stream
    call(cur)
    call(cur, small)
    torch.cuda.synchronize()
    eager = out.clone()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        call(cur)
        call(cur, small)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the calls changed the device's free memory"

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        call(stream.cuda_stream)
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(stream)
    for replay in range(3):
        out.fill_(float("nan"))
        call(cur, small)   # an eager call on the same array between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay}"

    # the size gate counts what the call's own layouts need: at 32768 x 16384 x 16384 row-major scales would be re-laid
    # into 25 MB of scratch (refused), scales already in MFMA32 order are read in place (served)
    bm, big = 32768, 16384
    g = torch.Generator(device=DEV).manual_seed(5)
    bx = torch.randint(0, 256, (bm, big // 2), dtype=torch.uint8, device=DEV, generator=g)
    bw = torch.randint(0, 256, (big, big // 2), dtype=torch.uint8, device=DEV, generator=g)
    bxs = torch.randint(122, 131, (bm, big // 32), dtype=torch.uint8, device=DEV, generator=g)   # any bytes, any order
    bws = torch.randint(122, 131, (big, big // 32), dtype=torch.uint8, device=DEV, generator=g)
    got = torch.empty(bm, big, dtype=torch.bfloat16, device=DEV)
    want = torch.empty(bm, big, dtype=torch.bfloat16, device=DEV)
    args = (bx.data_ptr(), bxs.data_ptr(), bw.data_ptr(), bws.data_ptr())
    assert lib.wave_mxfp4_gemm_static(*args, got.data_ptr(), bm, big, big, _lib.OUT_BF16, 0, 0, 0, 1, 0, cur) == _lib.ERR_WORKSPACE
    m32 = _lib.SCALE_MFMA32
    assert lib.wave_mxfp4_gemm_static(*args, got.data_ptr(), bm, big, big, _lib.OUT_BF16, m32, m32, 0, 1, 0, cur) == _lib.OK
    assert lib.wave_mxfp4_gemm(*args, want.data_ptr(), bm, big, big, _lib.OUT_BF16, m32, m32, 0, 1, None, 0, 0, cur) == _lib.OK
    torch.cuda.synchronize()
    assert torch.equal(got, want)
