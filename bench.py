"""Benchmark of the MXFP4 block-scaled GEMM on one MI355X.

One "step" is one GEMM of the headline workload (M = N = K = 8192, bf16 out,
seed 1, inputs resident in HBM).  Prints ONE JSON line: whole-job TFLOP/s, the
MFMA roofline of the tile kernel, the HBM roofline of the M = 16 decode shape
and the reference's CPU path (torch dequantise + f32 matmul) timed on a bounded
sample on this box's host cores.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3_m16|...]

Every timed leg is preceded by an untimed, time-based load of its own kernel
(launches until 50 ms of GPU time have passed, reported as `settle_ms`): the
GPU needs some tens of milliseconds of work to reach its steady clocks, so
without it a short --steps/--warmup reads up to 18 % slow.  `steps` and `warmup`
are then exactly what the caller passed.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MXFP4_TFLOPS = 10100.0   # MI355X dense FP4 MFMA
PEAK_HBM_GBPS = 8000.0        # MI355X HBM3E
PEAK_MXFP8_TFLOPS = 5000.0    # MI355X dense FP8 MFMA
SETTLE = {"ms": 50.0}        # untimed load in front of every timed leg (GPU milliseconds)
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.txt")

WORKLOADS = {
    # name: (m, n, k, out dtype, seed, scale range)
    "cfg1": (1024, 1024, 1024, "f32", 0, (124, 130)),
    "cfg2": (8192, 8192, 8192, "bf16", 1, (124, 130)),
    "cfg3_m1": (1, 28672, 8192, "bf16", 2, (120, 134)),
    "cfg3_m16": (16, 28672, 8192, "bf16", 2, (120, 134)),
    "cfg3_m32": (32, 28672, 8192, "bf16", 2, (120, 134)),
    "cfg3_m64": (64, 28672, 8192, "bf16", 2, (120, 134)),
    "cfg3_m128": (128, 28672, 8192, "bf16", 2, (120, 134)),
    "cfg3_m256": (256, 28672, 8192, "bf16", 2, (120, 134)),
    "cfg5": (4093, 6144, 7168, "f32", 4, (100, 154)),
}

# (M, N) pairs of the reference's benchmark shape list, all at K = 16000
# (wave_lang/kernel/wave/perf/mxfp4_shapes_macrotiles.csv, columns M,N,K; 103 distinct pairs)
REF_SHAPES_K = 16000
REF_SHAPES_MN = {
    512: [512, 1024, 2048, 8192],
    1024: [512, 1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 12288, 16384, 20480, 24576, 28672, 32768],
    1536: [8192],
    2048: [512, 1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 12288, 16384, 20480, 24576, 28672, 32768],
    2560: [8192],
    3072: [1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 12288, 16384, 20480],
    3584: [8192],
    4096: [1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 12288, 16384],
    4608: [8192],
    5120: [1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 12288],
    5632: [8192],
    6144: [1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192],
    6656: [8192],
    7168: [1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192],
    7680: [8192],
    8192: [512, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 4608, 5120, 5632, 6144, 6656, 7168, 7680, 8192],
}


def gemm_flops(m, n, k):
    return 2 * m * n * k


def gemm_bytes(m, n, k, out_bytes):
    return m * k // 2 + m * k // 32 + n * k // 2 + n * k // 32 + m * n * out_bytes


def make_gpu_inputs(torch, m, n, k, seed, scale_range, device, copies=1):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    lo, hi = scale_range
    sets = []
    for _ in range(copies):
        x = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
        w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
        xs = torch.randint(lo, hi + 1, (m, k // 32), dtype=torch.uint8, generator=g)
        ws = torch.randint(lo, hi + 1, (n, k // 32), dtype=torch.uint8, generator=g)
        sets.append(tuple(t.to(device) for t in (x, xs, w, ws)))
    return sets


def make_gpu_inputs_on_device(torch, m, n, k, scale_range, device, copies):
    """`copies` operand sets drawn on the GPU (uniform nibbles, scales in `scale_range`): for sweeps that rotate
    enough sets to keep B out of the 256 MB memory-side cache, where drawing on the host would dominate the run."""
    lo, hi = scale_range
    sets = []
    for _ in range(copies):
        sets.append((torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, device=device),
                     torch.randint(lo, hi + 1, (m, k // 32), dtype=torch.uint8, device=device),
                     torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=device),
                     torch.randint(lo, hi + 1, (n, k // 32), dtype=torch.uint8, device=device)))
    return sets


def settle(torch, run, min_ms=None):
    """Untimed clock-settle load: `run(n)` launches n of the leg's kernels; repeated until `min_ms` of GPU time have
    passed.  Returns the GPU milliseconds spent."""
    min_ms = SETTLE["ms"] if min_ms is None else min_ms
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    spent, n = 0.0, 4
    while spent < min_ms:
        e0.record()
        run(n)
        e1.record()
        torch.cuda.synchronize()
        dt = e0.elapsed_time(e1)
        spent += dt
        # aim each further chunk at about a fifth of the target
        n = max(1, min(4096, int(n * (min_ms / 5.0) / max(dt, 1e-3))))
    return spent


def timed(torch, run, steps, warmup):
    """settle, `warmup` untimed launches, then exactly `steps` launches between HIP events on the current stream
    (the stream the kernels are launched on).  Returns (wall seconds for all steps, seconds per launch from the
    events, settle milliseconds)."""
    settle_ms = settle(torch, run)
    run(warmup)
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    run(steps)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, ev0.elapsed_time(ev1) * 1e-3 / steps, settle_ms


def time_gemm(torch, wave_amd, sets, out, steps, warmup, **kw):
    """K launches back to back on the current stream; returns (wall seconds for
    all K, average seconds per launch from HIP events on that stream, settle ms)."""
    state = {"i": 0}

    def run(count):
        i = state["i"]
        for _ in range(count):
            x, xs, w, ws = sets[i % len(sets)]
            wave_amd.mxfp4_gemm(x, xs, w, ws, out, **kw)
            i += 1
        state["i"] = i

    return timed(torch, run, steps, warmup)


def read_traffic(workload):
    """HBM bytes per launch of the workload's dominant kernel (fetched + written) from the committed summary of
    the rocprofv3 FETCH_SIZE / WRITE_SIZE runs, or None when there is no line for it."""
    try:
        with open(TRAFFIC_FILE) as fh:
            for line in fh:
                f = line.split()
                if len(f) >= 4 and not line.startswith("#") and f[0] == workload:
                    return float(f[2]) + float(f[3])
    except OSError:
        pass
    return None


def write_traffic(workload, kernel_substr, fetch_csv, write_csv, fetch_factor, write_factor):
    """Updates the workload's line of profiles/hbm_traffic.txt from two rocprofv3 --pmc counter CSVs (FETCH_SIZE
    and WRITE_SIZE, KiB per dispatch) of the same bench command; the factors are bytes moved / bytes counted for
    the same counters on a device copy of known size (bench.py --copy-calibration)."""
    import csv

    def mean_kib(path, counter):
        vals = {}
        with open(path) as fh:
            for row in csv.DictReader(fh):
                if row["Counter_Name"] == counter and kernel_substr in row["Kernel_Name"]:
                    vals.setdefault(row.get("Dispatch_Id", len(vals)), 0.0)
                    vals[row.get("Dispatch_Id", len(vals) - 1)] += float(row["Counter_Value"])
        if not vals:
            raise SystemExit(f"{path}: no {counter} rows for a kernel matching {kernel_substr!r}")
        return sum(vals.values()) / len(vals)

    fetch = mean_kib(fetch_csv, "FETCH_SIZE") * 1024 * fetch_factor
    wrote = mean_kib(write_csv, "WRITE_SIZE") * 1024 * write_factor
    lines = []
    try:
        lines = [ln for ln in open(TRAFFIC_FILE).read().splitlines() if ln.split()[:1] != [workload]]
    except OSError:
        lines = ["# HBM bytes per launch of each workload's dominant kernel: rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE",
                 "# (KiB per dispatch, mean over the dispatches of `python3 bench.py --no-cpu --no-legs --steps 3 --warmup 1",
                 "# --workload <W>`), each scaled by the same counter on a 256 MiB device copy (--copy-calibration).",
                 "# Written by `python bench.py --workload <W> --write-traffic KERNEL,FETCH.csv,WRITE.csv,FETCH_FACTOR,WRITE_FACTOR`;",
                 "# read back into roofline.traffic.  Columns: workload kernel fetched_bytes written_bytes"]
    lines.append(f"{workload} {kernel_substr} {fetch:.4e} {wrote:.4e}")
    with open(TRAFFIC_FILE, "w") as fh:
        fh.write("\n".join(lines) + "\n")
    print(f"{TRAFFIC_FILE}: {lines[-1]}")


def cpu_baseline(torch, m, n, k, seed, scale_range, sample_rows):
    """The reference's CPU path (torch dequantise + f32 mm) on `sample_rows`
    rows of A against all of B, on this box's host cores."""
    from oracle.torch_oracle import torch_scaled_gemm_mxfp4

    cores = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    threads = min(cores, int(env)) if env and env.isdigit() else cores
    torch.set_num_threads(threads)
    rows = min(sample_rows, m)
    (x, xs, w, ws), = make_gpu_inputs(torch, rows, n, k, seed, scale_range, "cpu")
    torch_scaled_gemm_mxfp4(x[:8], w[:64], xs[:8], ws[:64])  # warm the thread pool
    # whole runs until about 10 s of CPU work are spent (at least 2, at most 8)
    runs, spent, deq, mm = 0, 0.0, 0.0, 0.0
    while runs < 2 or (spent < 10.0 and runs < 8):
        timings = {}
        t0 = time.perf_counter()
        torch_scaled_gemm_mxfp4(x, w, xs, ws, timings=timings)
        spent += time.perf_counter() - t0
        deq += timings["dequant_s"]
        mm += timings["matmul_s"]
        runs += 1
    dt = spent / runs
    return {
        "value": round(gemm_flops(rows, n, k) / dt / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"rows 0..{rows - 1} of A against all of B ({rows}x{n}x{k}), mean of {runs} runs after a warm-up",
        "seconds": round(dt, 3),
        "dequant_s": round(deq / runs, 3),
        "matmul_s": round(mm / runs, 3),
    }


def time_quantize(torch, wave_amd, rows, k, steps, warmup, device, shuffle=True):
    """(seconds per launch, algorithmic bytes, settle ms) of the bf16 -> MXFP4 quantiser on a [rows, k] activation;
    three inputs are rotated so that none is cache resident (402 MB together at 8192 x 8192)."""
    xs = [torch.randn(rows, k, device=device, dtype=torch.bfloat16) for _ in range(3)]
    lib = wave_amd._lib.load()
    q = torch.empty(rows, k // 2, dtype=torch.uint8, device=device)
    sc = torch.empty((rows + 31) // 32 * 32, (k // 32 + 7) // 8 * 8, dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream().cuda_stream
    layout = wave_amd._lib.SCALE_E8M0_SHUFFLE if shuffle else wave_amd._lib.SCALE_ROW_MAJOR
    state = {"i": 0}

    def run(count):
        for _ in range(count):
            st = lib.wave_mxfp4_quantize(xs[state["i"] % 3].data_ptr(), wave_amd._lib.IN_BF16, q.data_ptr(),
                                         sc.data_ptr(), rows, k, layout, stream)
            state["i"] += 1
            if st != 0:
                raise RuntimeError(f"wave_mxfp4_quantize: status {st}")

    _, per, settle_ms = timed(torch, run, steps, warmup)
    return per, rows * k * 2 + rows * k // 2 + rows * k // 32, settle_ms


def leg_moe_layer(torch, wave_amd, dev, steps_, warmup_, tokens=4096):
    """One mixture-of-experts MLP, the path of tests/kernel/moe_test.py:113-246 without its final weighted sum:
    routing table -> token alignment -> gathered quantiser -> grouped GEMM (gate and up projections) -> gated
    activation fused into the quantiser -> grouped GEMM (down projection).  Every scale tensor is written or kept in
    MFMA32 order, so no re-layout launch sits between the steps.  Returns the layer's time and that of each step."""
    from wave_amd import _lib as L

    topk, E, hidden, inter = 2, 8, 4096, 14336
    M32 = L.SCALE_MFMA32
    g = torch.Generator(device=dev).manual_seed(3)
    ids = torch.stack([torch.randperm(E, device=dev, generator=g)[:topk] for _ in range(tokens)]).to(torch.int32)
    n_ent = tokens * topk
    sorted_ids = torch.empty(n_ent, dtype=torch.int32, device=dev)
    expert_ids = torch.empty(n_ent, dtype=torch.int32, device=dev)
    total = torch.empty(1, dtype=torch.int32, device=dev)
    offs = torch.empty(E + 1, dtype=torch.int32, device=dev)
    act = torch.randn(tokens, hidden, device=dev, generator=g).to(torch.bfloat16)

    def to_m32(ws, n, k):
        return torch.stack([wave_amd.scale_convert(ws[e], n, k // 32, L.SCALE_ROW_MAJOR, M32) for e in range(E)])

    def weights(n, k):
        w = torch.randint(0, 256, (E, n, k // 2), dtype=torch.uint8, device=dev, generator=g)
        ws = torch.randint(120, 131, (E, n, k // 32), dtype=torch.uint8, device=dev, generator=g)
        return w, ws

    w1, w1s_rm = weights(2 * inter, hidden)
    w1s = to_m32(w1s_rm, 2 * inter, hidden)
    # the same weight with gate and up rows interleaved in blocks of 32 (once, outside the timed region): the order
    # the GEMM with the fused activation + quantiser takes
    w1_il = wave_amd.interleave_gate_up(w1)
    w1s_il = to_m32(wave_amd.interleave_gate_up(w1s_rm), 2 * inter, hidden)
    del w1s_rm
    w2, w2s_rm = weights(hidden, inter)
    w2s = to_m32(w2s_rm, hidden, inter)
    del w2s_rm
    h1 = torch.empty(n_ent, 2 * inter, dtype=torch.bfloat16, device=dev)
    out = torch.empty(n_ent, hidden, dtype=torch.bfloat16, device=dev)
    state = {}

    def step_align():
        wave_amd.moe_align_block_size(ids, E, 1, sorted_ids, expert_ids, total, offs)

    def step_gather():
        state["q1"], state["s1"] = wave_amd.quantize_mxfp4_rows(act, sorted_ids, topk, scale_layout=M32)

    def step_gemm1():
        wave_amd.mxfp4_gemm_grouped(state["q1"], state["s1"], w1, w1s, offs, h1, a_scale_layout=M32, b_scale_layout=M32)

    def step_act():
        state["q2"], state["s2"] = wave_amd.silu_and_mul_quantize(h1[:, :inter], h1[:, inter:], scale_layout=M32)

    def step_gemm2():
        wave_amd.mxfp4_gemm_grouped(state["q2"], state["s2"], w2, w2s, offs, out, a_scale_layout=M32, b_scale_layout=M32)

    def step_gemm1_fused():
        state["q2"], state["s2"] = wave_amd.mxfp4_gemm_gated_quantize(state["q1"], state["s1"], w1_il, w1s_il, offs,
                                                                     a_scale_layout=M32, b_scale_layout=M32)

    unfused = [("moe_align_block_size", step_align), ("gathered_quantiser", step_gather), ("grouped_gemm_gate_up", step_gemm1),
               ("gated_activation_quantiser", step_act), ("grouped_gemm_down", step_gemm2)]
    fused = [("moe_align_block_size", step_align), ("gathered_quantiser", step_gather),
             ("grouped_gemm_gate_up_activation_quantiser", step_gemm1_fused), ("grouped_gemm_down", step_gemm2)]
    flops = 2.0 * n_ent * (2 * inter) * hidden + 2.0 * n_ent * hidden * inter
    # what the layer has to move at least: both weights with their scales once, the activations in, the result out
    layer_bytes = E * (2 * inter * (hidden // 2 + hidden // 32) + hidden * (inter // 2 + inter // 32)) \
        + tokens * hidden * 2 + n_ent * hidden * 2

    def measure(steps):
        def layer(count):
            for _ in range(count):
                for _, fn in steps:
                    fn()

        layer(1)
        torch.cuda.synchronize()
        _, per_layer, _ = timed(torch, layer, steps_, warmup_)
        each = {}
        for name, fn in steps:
            def run(count, fn=fn):
                for _ in range(count):
                    fn()
            each[name] = round(timed(torch, run, steps_, warmup_)[1] * 1e6, 2)
        return {"layer_us": round(per_layer * 1e6, 2), "tflops": round(flops / per_layer / 1e12, 1),
                "frac_of_mxfp4_peak": round(flops / per_layer / 1e12 / PEAK_MXFP4_TFLOPS, 4),
                "gb_per_s": round(layer_bytes / per_layer / 1e9, 1),
                "frac_of_hbm_peak": round(layer_bytes / per_layer / 1e9 / PEAK_HBM_GBPS, 4), "steps_us": each,
                "sum_of_steps_us": round(sum(each.values()), 2)}

    # the layer as the library runs it best: activation and quantiser in the first GEMM's C write; and the chain of
    # separate kernels it replaces (the reference's: tests/kernel/moe_test.py:113-129)
    leg = {"workload": f"moe_layer: {tokens} tokens x top-{topk} of {E} experts, hidden {hidden}, intermediate {inter}; "
                       "gate/up GEMM with the gated activation and the quantiser fused into its output",
           "algorithmic_bytes": layer_bytes, "rows_per_expert": n_ent / E}
    try:
        leg.update(measure(fused))
    except (RuntimeError, ValueError) as e:
        # (a serving batch: fewer 256x256 tiles than workgroups, the fused first GEMM is not taken; the chain of
        # separate kernels below is what runs)
        if "unsupported" not in str(e):
            raise
        leg["workload"] = leg["workload"].split(";")[0] + "; separate kernels (the batch is too small for the fused first GEMM)"
    leg["separate_activation_kernel"] = measure(unfused)
    if "layer_us" not in leg:
        leg.update(leg["separate_activation_kernel"])
    return leg


def leg_cfg4(torch, wave_amd, dev, steps, warmup, variant=0):
    """The grouped (MoE) GEMM of cfg4: E = 8 experts, 4096 tokens x top-2 = 8192 rows dealt multinomially, rows
    sorted by expert, N = 14336, K = 4096, bf16 out, seed 3."""
    import numpy as np

    from wave_amd import _lib as L

    E, n, k, rows = 8, 14336, 4096, 8192
    counts = np.random.default_rng(3).multinomial(rows, np.ones(E) / E)
    offs = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).to(dev)
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8, device=dev, generator=g)
    xs = torch.randint(124, 131, (rows, k // 32), dtype=torch.uint8, device=dev, generator=g)
    w = torch.randint(0, 256, (E, n, k // 2), dtype=torch.uint8, device=dev, generator=g)
    ws = torch.randint(124, 131, (E, n, k // 32), dtype=torch.uint8, device=dev, generator=g)
    out = torch.empty(rows, n, dtype=torch.bfloat16, device=dev)

    def run(count):
        for _ in range(count):
            wave_amd.mxfp4_gemm_grouped(x, xs, w, ws, offs, out, variant=variant)

    wall, per, settle_ms = timed(torch, run, steps, warmup)
    # resident expert weights: their scales converted to the MFMA operand order once, outside the timed region
    ws32 = torch.stack([wave_amd.scale_convert(ws[e], n, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32) for e in range(E)])

    def run32(count):
        for _ in range(count):
            wave_amd.mxfp4_gemm_grouped(x, xs, w, ws32, offs, out, b_scale_layout=L.SCALE_MFMA32, variant=variant)

    _, per32, _ = timed(torch, run32, steps, warmup)
    flops = 2.0 * rows * n * k
    # the same experts at a serving batch: 64 tokens x top-2 = 128 rows dealt multinomially; every expert's B is
    # read once for a handful of rows, so the call is bound by HBM (two copies of the weights rotated: 500 MB)
    srows = 128
    scounts = np.random.default_rng(3).multinomial(srows, np.ones(E) / E)
    soffs = torch.from_numpy(np.concatenate([[0], np.cumsum(scounts)]).astype(np.int32)).to(dev)
    wsets = [(w, ws), (w.clone(), ws.clone())]
    sout = torch.empty(srows, n, dtype=torch.bfloat16, device=dev)
    state = {"i": 0}

    def run_serving(count):
        for _ in range(count):
            wi, wsi = wsets[state["i"] & 1]
            state["i"] += 1
            wave_amd.mxfp4_gemm_grouped(x[:srows], xs[:srows], wi, wsi, soffs, sout, variant=variant)

    _, pers, _ = timed(torch, run_serving, steps, warmup)
    sbytes = srows * (k // 2 + k // 32) + E * n * (k // 2 + k // 32) + srows * n * 2
    del wsets
    return {"workload": f"cfg4: E={E} N={n} K={k} rows={rows} (counts {counts.tolist()}) bf16 out seed 3",
            "kernel": "persist_gemm_kernel (grouped)", "launch_us": round(per * 1e6, 2),
            "tflops": round(flops / per / 1e12, 1), "frac_of_mxfp4_peak": round(flops / per / 1e12 / PEAK_MXFP4_TFLOPS, 4),
            "settle_ms": round(settle_ms, 1), "wall_s_per_step": wall / steps,
            "resident_weight_scales": {"workload": "the same call with the experts' B scales already in MFMA operand order",
                                       "launch_us": round(per32 * 1e6, 2), "tflops": round(flops / per32 / 1e12, 1),
                                       "frac_of_mxfp4_peak": round(flops / per32 / 1e12 / PEAK_MXFP4_TFLOPS, 4)},
            "serving_batch": {"workload": f"the same experts, {srows} rows (counts {scounts.tolist()}), weights from HBM",
                              "kernel": "mid_gemm_kernel (grouped)", "launch_us": round(pers * 1e6, 2),
                              "algorithmic_bytes": sbytes, "gb_per_s": round(sbytes / pers / 1e9, 1),
                              "frac_of_hbm_peak": round(sbytes / pers / 1e9 / PEAK_HBM_GBPS, 4)}}


def leg_mxfp8(torch, wave_amd, dev, steps, warmup, variant=0):
    """tests/kernel/wave_gemm_mxfp_test.py:416-501 at its larger shape: e5m2 operands, scales 124..127, f32 out."""
    m = n = k = 8192
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(m, k, device=dev, generator=g).to(torch.float8_e5m2)
    w_t = torch.randn(n, k, device=dev, generator=g).to(torch.float8_e5m2)
    xs = torch.randint(124, 128, (m, k // 32), dtype=torch.uint8, device=dev, generator=g)
    ws = torch.randint(124, 128, (n, k // 32), dtype=torch.uint8, device=dev, generator=g)
    out = torch.empty(m, n, dtype=torch.float32, device=dev)

    def run(count):
        for _ in range(count):
            wave_amd.mxfp8_gemm(x, xs, w_t, ws, out, variant=variant)

    wall, per, settle_ms = timed(torch, run, steps, warmup)
    flops = 2.0 * m * n * k
    # the same activations against packed MXFP4 weights (8-bit x 4-bit operands of the scaled MFMA)
    from wave_amd import _lib as L
    w4 = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=g)

    def run_mixed(count):
        for _ in range(count):
            wave_amd.mxfp8_gemm(x, xs, w4, ws, out, elem_format=(L.MXFP8_E5M2, L.MXFP8_B_E2M1), variant=variant)

    _, mper, _ = timed(torch, run_mixed, steps, warmup)
    w4p = wave_amd.b_preshuffle(w4)
    del w4

    def run_mixed_pre(count):
        for _ in range(count):
            wave_amd.mxfp8_gemm(x, xs, w4p, ws, out, elem_format=(L.MXFP8_E5M2, L.MXFP8_B_E2M1), b_preshuffled=True)

    _, mpper, _ = timed(torch, run_mixed_pre, steps, warmup)
    del w4p
    # the same problem with B in the library's preshuffled 8-bit order (B straight into registers), scales as the
    # call above hands them over (row-major, re-laid out by a launch of the call) and resident in MFMA32 order;
    # and both kernels on zero operands (no switching power: what the schedules reach at the full clock)
    wp = wave_amd.mxfp8_b_preshuffle(w_t)

    def run_pre(count):
        for _ in range(count):
            wave_amd.mxfp8_gemm(x, xs, wp, ws, out, b_preshuffled=True)

    _, pper, _ = timed(torch, run_pre, steps, warmup)
    xs32 = wave_amd.scale_convert(xs, m, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32)
    ws32 = wave_amd.scale_convert(ws, n, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32)

    def run_pre32(count):
        for _ in range(count):
            wave_amd.mxfp8_gemm(x, xs32, wp, ws32, out, b_preshuffled=True, a_scale_layout=L.SCALE_MFMA32,
                                b_scale_layout=L.SCALE_MFMA32, workspace=False)

    _, pper32, _ = timed(torch, run_pre32, steps, warmup)
    del wp
    z = torch.zeros(m, k, dtype=torch.float8_e5m2, device=dev)

    def run_zero(count):
        for _ in range(count):
            wave_amd.mxfp8_gemm(z, xs, z, ws, out, variant=variant)

    def run_zero_pre(count):
        for _ in range(count):
            wave_amd.mxfp8_gemm(z, xs, z, ws, out, b_preshuffled=True)

    _, zper, _ = timed(torch, run_zero, max(steps // 2, 5), max(warmup // 2, 3))
    _, zpper, _ = timed(torch, run_zero_pre, max(steps // 2, 5), max(warmup // 2, 3))

    def rate(t):
        return {"launch_us": round(t * 1e6, 2), "tflops": round(flops / t / 1e12, 1),
                "frac_of_mxfp8_peak": round(flops / t / 1e12 / PEAK_MXFP8_TFLOPS, 4)}

    pre = dict(rate(pper), workload="the same problem, B in wave_mxfp8_b_preshuffle order (B-direct kernel), per call "
                                    "with the launch that re-lays the row-major scales out",
               kernel="asym8_gemm_kernel", resident_scales=rate(pper32),
               e5m2_x_e2m1=dict(rate(mpper), workload="8-bit activations against MXFP4 weights in b_preshuffle order"),
               zero_operands={"symmetric_us": round(zper * 1e6, 2), "b_direct_us": round(zpper * 1e6, 2)})
    return {"workload": f"mxfp8: M={m} N={n} K={k} e5m2 x e5m2, f32 out, seed 5", "kernel": "persist_gemm_fp8_kernel",
            "b_preshuffled": pre,
            "launch_us": round(per * 1e6, 2), "tflops": round(flops / per / 1e12, 1),
            "frac_of_mxfp8_peak": round(flops / per / 1e12 / PEAK_MXFP8_TFLOPS, 4), "settle_ms": round(settle_ms, 1),
            "e5m2_x_e2m1": {"workload": "the same activations against MXFP4 weights [N, K/2]",
                            "launch_us": round(mper * 1e6, 2), "tflops": round(flops / mper / 1e12, 1),
                            "frac_of_mxfp8_peak": round(flops / mper / 1e12 / PEAK_MXFP8_TFLOPS, 4)},
            "wall_s_per_step": wall / steps}


def leg_dense(torch, wave_amd, dev, name, steps, warmup, variant=0):
    """One of the dense WORKLOADS through the library's own kernel choice."""
    m, n, k, od, seed, srange = WORKLOADS[name]
    sets = make_gpu_inputs(torch, m, n, k, seed, srange, dev, copies=1)
    out = torch.empty(m, n, dtype=torch.bfloat16 if od == "bf16" else torch.float32, device=dev)
    _, per, settle_ms = time_gemm(torch, wave_amd, sets, out, steps, warmup, variant=variant)
    flops = gemm_flops(m, n, k)
    leg = {"workload": f"{name}: M={m} N={n} K={k} {od} out seed {seed}", "launch_us": round(per * 1e6, 2),
           "tflops": round(flops / per / 1e12, 1), "frac_of_mxfp4_peak": round(flops / per / 1e12 / PEAK_MXFP4_TFLOPS, 4),
           "settle_ms": round(settle_ms, 1)}
    if variant == 0 and k % 256 == 0:
        # the same call with both scale tensors in the reference's e8m0_shuffle order (read in place)
        from wave_amd import _lib as L
        x, xs, w, ws = sets[0]
        xsh = wave_amd.scale_convert(xs, m, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_E8M0_SHUFFLE)
        wsh = wave_amd.scale_convert(ws, n, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_E8M0_SHUFFLE)
        _, sper, _ = time_gemm(torch, wave_amd, [(x, xsh, w, wsh)], out, steps, warmup,
                               a_scale_layout=L.SCALE_E8M0_SHUFFLE, b_scale_layout=L.SCALE_E8M0_SHUFFLE)
        leg["e8m0_shuffled_scales"] = {"launch_us": round(sper * 1e6, 2), "tflops": round(flops / sper / 1e12, 1),
                                       "frac_of_mxfp4_peak": round(flops / sper / 1e12 / PEAK_MXFP4_TFLOPS, 4)}
    return leg


def mfma_ceiling(torch, dev, steps, warmup, compact=False):
    """What the matrix pipes sustain on the scaled FP4 MFMA alone (wave_amd/csrc/mfma_probe.hip): random operand
    bytes against zeros, 4 and 8 waves per CU, one workgroup per CU.  compact: the 8-wave shape of the GEMM kernels
    only, random and zeros, no duty-cycle rows (the leg of the default line)."""
    import ctypes

    path = os.path.join(ROOT, "wave_amd", "csrc", "libwave_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `make -C wave_amd/csrc`")
    probe = ctypes.CDLL(path)
    vp, i32 = ctypes.c_void_p, ctypes.c_int
    probe.wave_probe_mfma_fp4.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
    probe.wave_probe_mfma_fp4.restype = i32
    probe.wave_probe_mfma_fp4_duty.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, vp]
    probe.wave_probe_mfma_fp4_duty.restype = i32
    probe.wave_probe_operand_bytes.argtypes = [i32, i32]
    probe.wave_probe_operand_bytes.restype = ctypes.c_size_t
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    stream = torch.cuda.current_stream().cuda_stream
    iters = 8000   # x 32 MFMAs x 32 cycles per wave: about 4 ms per launch at one wave per SIMD
    rows = []
    for waves in ((8,) if compact else (4, 8)):
        nbytes = probe.wave_probe_operand_bytes(cus, waves)
        g = torch.Generator(device=dev).manual_seed(11)
        operands = {"random": torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=dev, generator=g),
                    "zeros": torch.zeros(nbytes, dtype=torch.uint8, device=dev)}
        out = torch.empty(cus * waves * 64, dtype=torch.float32, device=dev)
        ticks = torch.empty(cus, dtype=torch.int64, device=dev)
        # idle: s_sleep 1 instructions after every 32 MFMAs (4 waves per CU only): the pipes' duty cycle as a knob
        for data, idle in [("random", 0), ("zeros", 0)] + ([("random", s) for s in (4, 8, 16)] +
                                                           [("zeros", s) for s in (4, 8, 16)] if waves == 4 else []):
            src = operands[data]

            def run(count):
                for _ in range(count):
                    rc = probe.wave_probe_mfma_fp4_duty(src.data_ptr(), out.data_ptr(), ticks.data_ptr(), iters, 110,
                                                        cus, waves, idle, stream)
                    if rc != 0:
                        raise RuntimeError(f"wave_probe_mfma_fp4_duty: {rc}")

            _, per, settle_ms = timed(torch, run, 5 if compact else max(steps // 10, 10), 2 if compact else max(warmup // 10, 2))
            mfmas_per_wave = iters * 32
            flops = cus * waves * mfmas_per_wave * 2.0 * 32 * 32 * 64
            # MFMA cycles each SIMD has to issue (32 per instruction, waves / 4 waves per SIMD): the clock if the pipe
            # never idles, a lower bound of it otherwise
            clock_ghz = mfmas_per_wave * 32 * (waves / 4) / per / 1e9
            rows.append({"operands": data, "waves_per_cu": waves, "idle_sleeps_per_32_mfma": idle, "launch_ms": round(per * 1e3, 3),
                         "tflops": round(flops / per / 1e12, 1),
                         "frac_of_mxfp4_peak": round(flops / per / 1e12 / PEAK_MXFP4_TFLOPS, 4),
                         "mfma_clock_ghz": round(clock_ghz, 3), "settle_ms": round(settle_ms, 1)})
    best_random = max(r["tflops"] for r in rows if r["operands"] == "random" and r["idle_sleeps_per_32_mfma"] == 0)
    return rows, best_random


def read_once_probe(torch, dev, steps, warmup):
    """A read-once stream of 117 MB (the decode shapes' B: 224 strips of 128 rows x 4 KB) with nothing else going
    on (wave_amd/csrc/mfma_probe.hip, stream_probe_kernel): from HBM (three sets rotated) and from the Infinity
    Cache (one set)."""
    import ctypes

    probe = ctypes.CDLL(os.path.join(ROOT, "wave_amd", "csrc", "libwave_probe.so"))
    vp, i32 = ctypes.c_void_p, ctypes.c_int
    probe.wave_probe_read_once.argtypes = [vp, i32, vp, vp]
    probe.wave_probe_read_once.restype = i32
    stream = torch.cuda.current_stream().cuda_stream
    strips, set_bytes = 224, 224 * 128 * 4096
    src = torch.randint(0, 256, (3 * set_bytes,), dtype=torch.uint8, device=dev)
    sink = torch.zeros(16, dtype=torch.int32, device=dev)
    rows = []
    for name, nsets in (("hbm (3 sets rotated)", 3), ("infinity cache (1 set)", 1)):
        state = {"i": 0}

        def run(count):
            for _ in range(count):
                rc = probe.wave_probe_read_once(src.data_ptr() + (state["i"] % nsets) * set_bytes, strips,
                                                sink.data_ptr(), stream)
                state["i"] += 1
                if rc != 0:
                    raise RuntimeError(f"wave_probe_read_once: {rc}")

        _, per, _ = timed(torch, run, max(steps, 100), max(warmup, 30))
        rows.append({"source": name, "bytes": set_bytes, "launch_us": round(per * 1e6, 2),
                     "tb_per_s": round(set_bytes / per / 1e12, 2)})
    return rows


def l2_dma_probe(torch, dev, steps, warmup):
    """What L2 and Infinity Cache deliver to the CUs' LDS through the GEMM kernels' operand DMA alone
    (wave_amd/csrc/mfma_probe.hip, dma_probe_kernel): 12 panels of 1 MB (3 per XCD, L2 resident) and 96 (12 MB per
    XCD: from the Infinity Cache)."""
    import ctypes

    probe = ctypes.CDLL(os.path.join(ROOT, "wave_amd", "csrc", "libwave_probe.so"))
    vp, i32 = ctypes.c_void_p, ctypes.c_int
    probe.wave_probe_l2_dma.argtypes = [vp, i32, i32, i32, vp]
    probe.wave_probe_l2_dma.restype = i32
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    stream = torch.cuda.current_stream().cuda_stream
    src = torch.randint(0, 256, (96 << 20,), dtype=torch.uint8, device=dev)
    iters, rows = 64, []
    for panels in (12, 96):
        def run(count):
            for _ in range(count):
                rc = probe.wave_probe_l2_dma(src.data_ptr(), panels, iters, cus, stream)
                if rc != 0:
                    raise RuntimeError(f"wave_probe_l2_dma: {rc}")

        _, per, _ = timed(torch, run, max(steps // 30, 5), max(warmup // 30, 2))
        rows.append({"panels_of_1mb": panels, "footprint_per_xcd_mb": panels * 8 // 32 if panels < 32 else panels // 8,
                     "launch_ms": round(per * 1e3, 3), "tb_per_s": round(cus * iters * (1 << 20) / per / 1e12, 2)})
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100, help="untimed launches in front of the timed ones (after the "
                    "time-based settle load every leg runs anyway)")
    ap.add_argument("--workload", default="cfg2",
                    choices=sorted(WORKLOADS) + ["cfg4", "quant_bf16", "mxfp8", "moe_glue", "ref_shapes", "mfma_ceiling",
                                                 "decode_sweep", "moe_serving", "moe_layer", "tile_choice"],
                    help="cfg*: the GEMM configurations; quant_bf16: the activation quantiser alone on the "
                         "8192 x 8192 bf16 activation of cfg2; mxfp8: the MXFP8 (e5m2) GEMM at 8192^3, f32 out; "
                         "cfg4: the grouped (MoE) GEMM, 8 experts, 8192 rows, N=14336, K=4096; moe_glue: the steps around "
                         "it at the same sizes (token alignment, gathered quantiser, gated activation + quantiser); "
                         "ref_shapes: the reference's benchmark shape list; mfma_ceiling: the scaled FP4 MFMA alone, "
                         "random operands against zeros (the power-limited ceiling of the matrix pipes); decode_sweep: "
                         "M = 1 .. 256 against wide weights from HBM, every kernel that serves the shape beside the "
                         "library's own choice; moe_serving: the grouped GEMM at serving batches, experts x rows per "
                         "expert, the mid-M kernel beside the tile kernels; moe_layer: one mixture-of-experts MLP end to end "
                         "(alignment, gathered quantiser, grouped GEMM, gated quantiser, grouped GEMM), step by step and whole; "
                         "tile_choice: the library's own choice against every tile shape, split and the mid-M kernel by name "
                         "on random mid-size shapes with the weights from HBM (--steps: number of shapes, default 60)")
    ap.add_argument("--variant", type=int, default=0, help="kernel variant of include/wave_mxfp4.h (0 = auto)")
    ap.add_argument("--resident-scales", action="store_true",
                    help="decode_sweep: both scale tensors handed over in MFMA32 order (no re-layout launch for any kernel)")
    ap.add_argument("--preshuffled-b", action="store_true", help="decode_sweep: B in b_preshuffle order")
    ap.add_argument("--moe-tokens", type=int, default=4096, help="moe_layer: tokens per call (top-2 of 8 experts)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-legs", "--no-decode", dest="no_legs", action="store_true",
                    help="cfg2 only: skip the legs beside the headline (decode shapes, quantiser, cfg4, cfg5, mxfp8)")
    ap.add_argument("--cpu-rows", type=int, default=8192,
                    help="rows of A in the CPU baseline leg (default: the whole workload)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="instead of a GEMM, run device-to-device copies of 256 MiB (the known-size kernel "
                         "that hardware byte counters are scaled by) and print their size")
    ap.add_argument("--write-traffic", metavar="KERNEL,FETCH_CSV,WRITE_CSV,FETCH_FACTOR,WRITE_FACTOR",
                    help="no GPU work: update this workload's line of profiles/hbm_traffic.txt from two rocprofv3 "
                         "--pmc counter CSVs of this command")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this operator runs on one GPU; --gpus N with N > 1 is not supported "
              "(the operator shards over GPUs by splitting N or M, with no exchange between them)", file=sys.stderr)
        sys.exit(2)
    if args.write_traffic:
        kernel, fetch_csv, write_csv, ff, wf = args.write_traffic.split(",")
        write_traffic(args.workload, kernel, fetch_csv, write_csv, float(ff), float(wf))
        return

    import torch

    import wave_amd
    from wave_amd import _lib

    _lib.load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = "cuda:0"
    torch.cuda.set_device(0)
    common = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
              "vs_baseline": None}

    if args.copy_calibration:
        nbytes = 256 << 20
        src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": True, "bytes_read_per_launch": nbytes,
                          "bytes_written_per_launch": nbytes, "launches": args.warmup + args.steps}))
        return

    if args.workload == "mfma_ceiling":
        rows, best = mfma_ceiling(torch, dev, args.steps, args.warmup)
        # the GEMM kernels themselves at 8192^3 on the seeded random operands and on all-zero operands (scales in
        # MFMA order, no pre-pass): the same instruction stream and memory traffic, only the power per instruction
        # differs; and with B preshuffled, the B-direct kernel
        from wave_amd import _lib as L
        gm = gn = gk = 8192
        (gx, gxs, gw, gws), = make_gpu_inputs(torch, gm, gn, gk, 1, (124, 130), dev)
        gxs = wave_amd.scale_convert(gxs, gm, gk // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32)
        gws = wave_amd.scale_convert(gws, gn, gk // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32)
        gout = torch.empty(gm, gn, dtype=torch.bfloat16, device=dev)
        gemm_rows = []
        for kernel, b_layout, bmat in (("persist_gemm_kernel", L.B_ROW_MAJOR, gw),
                                       ("asym_gemm_kernel", L.B_PRESHUFFLE, wave_amd.b_preshuffle(gw))):
            for data, xa, wb in (("random", gx, bmat), ("zeros", torch.zeros_like(gx), torch.zeros_like(bmat))):
                _, per, settle_ms = time_gemm(torch, wave_amd, [(xa, gxs, wb, gws)], gout, args.steps, args.warmup,
                                              a_scale_layout=L.SCALE_MFMA32, b_scale_layout=L.SCALE_MFMA32,
                                              b_layout=b_layout)
                tf = gemm_flops(gm, gn, gk) / per / 1e12
                gemm_rows.append({"kernel": kernel, "operands": data, "launch_us": round(per * 1e6, 2),
                                  "tflops": round(tf, 1), "frac_of_mxfp4_peak": round(tf / PEAK_MXFP4_TFLOPS, 4),
                                  "frac_of_mfma_alone": round(tf / max(r["tflops"] for r in rows if r["operands"] == data), 4),
                                  "settle_ms": round(settle_ms, 1)})
        print(json.dumps(dict(common, **{
            "metric": "scaled FP4 MFMA alone (v_mfma_scale_f32_32x32x64_f8f6f4, no memory traffic), TFLOP/s on random operands",
            "value": best, "unit": "TFLOP/s", "ms_per_step": min(r["launch_ms"] for r in rows if r["operands"] == "random"),
            "dtype": "mxfp4 (e2m1 x e8m0) in, f32 accumulate", "data": "synthetic (uniform random bytes / zeros)",
            "config": {"workload": "mfma_ceiling: one workgroup per CU, 4 or 8 waves, 8000 x 32 MFMAs per wave and launch"},
            "roofline": {"bound": "mfma", "achieved": best, "peak": PEAK_MXFP4_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(best / PEAK_MXFP4_TFLOPS, 4), "traffic": None, "kernel": "mfma_probe_kernel"},
            "runs": rows, "gemm_8192": gemm_rows,
            "operand_dma_alone": l2_dma_probe(torch, dev, args.steps, args.warmup),
            "read_once_stream": read_once_probe(torch, dev, args.steps, args.warmup)})))
        return

    if args.workload == "quant_bf16":
        rows, k = 8192, 8192
        qper, qbytes, settle_ms = time_quantize(torch, wave_amd, rows, k, args.steps, args.warmup, dev)
        gbps = qbytes / qper / 1e9
        print(json.dumps(dict(common, **{
            "metric": "activation quantiser, GB/s % HBM", "value": round(gbps, 1), "unit": "GB/s",
            "ms_per_step": round(qper * 1e3, 4), "dtype": "bf16 in, e2m1 + e8m0 out", "data": "synthetic (normal)",
            "settle_ms": round(settle_ms, 1),
            "config": {"workload": f"quant_bf16: bf16 [{rows}, {k}] -> MXFP4, scales in e8m0_shuffle order, "
                                   "3 inputs rotated"},
            "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                         "frac": round(gbps / PEAK_HBM_GBPS, 4), "traffic": read_traffic("quant_bf16"),
                         "kernel": "quantize_kernel", "launch_us": round(qper * 1e6, 2)}})))
        return

    if args.workload == "tile_choice":
        # The library's own choice of tile shape, split along K and kernel against every candidate asked for by
        # name, on shapes drawn at random from the range where it chooses by duration estimates (more than 64 rows,
        # N = 2048..32768, K >= 3584 in whole K tiles, at most two rounds of 256x256 tiles; drawn here up to 15360).  Operand sets are
        # rotated past the 256 MB memory-side cache, so B comes from HBM as a model's weights do; bf16 out; either
        # scale layout.  Every timing is the best of two; the library's choice is timed last.
        import math
        import numpy as np
        from wave_amd import _lib as L

        SETTLE["ms"] = 5.0
        rng = np.random.default_rng(5)
        names = [("mid", L.VARIANT_MID_M), ("t128", L.VARIANT_T128x128_W2x2), ("t128x256", L.VARIANT_T128x256_W2x2),
                 ("t256w8", L.VARIANT_T256x256_W4x2)]
        rows = []
        count = 60 if args.steps == 300 else args.steps
        while len(rows) < count:
            m = int(2 ** rng.uniform(6.1, 11.6))
            n = 128 * int(rng.integers(16, 121))
            k = 256 * int(rng.integers(14, 65))
            native = bool(rng.integers(0, 2))
            if ((m + 255) // 256) * ((n + 255) // 256) > 512:
                continue
            copies = max(2, min(80, math.ceil(400e6 / (n * k / 2))))
            sets = make_gpu_inputs_on_device(torch, m, n, k, (120, 134), dev, copies)
            if native:
                sets = [(x, wave_amd.scale_convert(xs, m, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32), w,
                         wave_amd.scale_convert(ws, n, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32)) for x, xs, w, ws in sets]
            kw = dict(a_scale_layout=L.SCALE_MFMA32, b_scale_layout=L.SCALE_MFMA32) if native else {}
            out = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
            iters = max(16, copies)

            def best_of_two(**opts):
                return min(time_gemm(torch, wave_amd, sets, out, iters, 4, **opts, **kw)[1] for _ in range(2)) * 1e6

            by_name = {}
            for name, v in names:
                for split in (0, 1, 2, 4, 8):
                    if name == "mid" and (split or m > 256):
                        continue
                    try:
                        by_name[f"{name}/{split}"] = round(best_of_two(variant=v, split_k=split), 1)
                    except (RuntimeError, ValueError):
                        pass   # (a split this K does not divide into, or a kernel that does not take the shape)
            auto = round(best_of_two(variant=L.VARIANT_AUTO, split_k=0), 1)
            best = min(by_name, key=by_name.get)
            rows.append({"m": m, "n": n, "k": k, "mfma32_scales": native, "auto_us": auto, "best": best,
                         "best_us": by_name[best], "ratio": round(auto / by_name[best], 3)})
            del sets, out
        ratios = [r["ratio"] for r in rows]
        print(json.dumps(dict(common, **{
            "metric": "library's choice / best kernel by name, geometric mean over random mid-size shapes",
            "value": round(math.exp(sum(math.log(r) for r in ratios) / len(ratios)), 4), "unit": "ratio",
            "higher_is_better": False,
            "ms_per_step": round(sum(r["auto_us"] for r in rows) * 1e-3, 3),
            "dtype": "mxfp4 (e2m1 x e8m0) in, f32 accumulate, bf16 out",
            "data": "synthetic (uniform nibbles, scales 120..134), operand sets rotated past the memory-side cache",
            "config": {"workload": f"tile_choice: {len(rows)} shapes, M 68..3100, N 2048..15360, K 3584..16384, seed 5"},
            "within_5_percent": sum(r <= 1.05 for r in ratios), "within_10_percent": sum(r <= 1.10 for r in ratios),
            "worst": max(ratios), "shapes": rows})))
        return

    if args.workload == "decode_sweep":
        # M x N x K against weights that come from HBM (operand sets rotated), bf16 out: the library's own choice
        # beside the streaming kernel (M <= 64), the mid-M kernel and the best tile kernel, each asked for by name
        from wave_amd import _lib as L

        SETTLE["ms"] = 20.0
        rows = []
        # --resident-scales: both scale tensors handed over in MFMA32 order (static weights, activations from the
        # quantiser), where no kernel needs a re-layout launch and the library's choice follows other borders;
        # --preshuffled-b on top: B in b_preshuffle order, the B-direct mid-M kernel among the candidates
        resident, pre = args.resident_scales, args.preshuffled_b
        grid_n = (12288, 14336, 20480, 28672, 40960, 57344) if resident else (8192, 14336, 28672, 57344)
        grid_m = (16, 32, 48, 64, 96, 128, 192, 256) if resident else (1, 16, 32, 64, 128, 256)
        kw = {}
        if resident:
            kw.update(a_scale_layout=L.SCALE_MFMA32, b_scale_layout=L.SCALE_MFMA32)
        if pre:
            kw.update(b_layout=L.B_PRESHUFFLE)
        for k in (8192, 4096):
            for n in grid_n:
                for m in grid_m:
                    # (at least 400 MB of B in rotation: beyond the 256 MB memory-side cache at every shape)
                    copies = max(2, -(-400_000_000 // (n * k // 2)))
                    sets = make_gpu_inputs_on_device(torch, m, n, k, (120, 134), dev, copies)
                    if resident or pre:
                        sets = [(x, wave_amd.scale_convert(xs, m, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32) if resident else xs,
                                 wave_amd.b_preshuffle(w) if pre else w,
                                 wave_amd.scale_convert(ws, n, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32) if resident else ws)
                                for x, xs, w, ws in sets]
                    out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
                    us = {}
                    names = [("mid", L.VARIANT_MID_M, 1)]
                    if m <= 64:
                        names.append(("stream", L.VARIANT_SKINNY, 1))
                    if m > 64 or (resident and m >= 32):
                        names += [("t128x128", L.VARIANT_T128x128_W2x2, 0), ("t128x256", L.VARIANT_T128x256_W2x2, 0),
                                  ("t256x256", L.VARIANT_T256x256_W4x2, 0)]
                    if pre and k % (2048 if m <= 128 else 1024) == 0:
                        names.append(("midb", L.VARIANT_MID_M_BDIRECT, 1))
                    # (the library's choice is timed first and last and the shorter time kept: right behind the
                    # power-hungry tile kernels the same launch reads up to 5 % long)
                    names = [("auto", L.VARIANT_AUTO, 0)] + names + [("auto", L.VARIANT_AUTO, 0)]
                    for name, v, split in names:
                        _, per, _ = time_gemm(torch, wave_amd, sets, out, min(args.steps, 100), 20, variant=v, split_k=split, **kw)
                        us[name] = min(us.get(name, 1e9), round(per * 1e6, 2))
                    nbytes = gemm_bytes(m, n, k, 2)
                    rows.append({"m": m, "n": n, "k": k, "us": us, "bytes": nbytes,
                                 "auto_frac_of_hbm_peak": round(nbytes / (us["auto"] * 1e-6) / 1e9 / PEAK_HBM_GBPS, 4)})
                    del sets, out
        worst = max(r["us"]["auto"] / min(r["us"].values()) for r in rows)
        print(json.dumps(dict(common, **{
            "metric": "MXFP4 GEMM at decode shapes: worst ratio of the library's choice to the best kernel",
            "value": round(worst, 3), "unit": "x", "higher_is_better": False,
            "ms_per_step": round(sum(r["us"]["auto"] for r in rows) * 1e-3, 3),
            "dtype": "mxfp4 (e2m1 x e8m0) in, f32 accumulate, bf16 out",
            "data": "synthetic (seeded uniform nibbles and scales), weights from HBM",
            "config": {"workload": f"decode_sweep: {len(rows)} shapes M x N x K, bf16 out, seed 2" +
                       (", both scale tensors in MFMA32 order" if resident else ", row-major scales") +
                       (", B in b_preshuffle order" if pre else "")}, "shapes": rows})))
        return

    if args.workload == "moe_serving":
        # the grouped GEMM at serving batches: E experts x rows per expert (even groups and multinomially dealt ones),
        # weights from HBM (three copies rotated), bf16 out; the library's choice beside the mid-M kernel and the
        # table-driven tile kernels asked for by name
        import numpy as np
        from wave_amd import _lib as L

        SETTLE["ms"] = 20.0
        g = torch.Generator(device="cpu").manual_seed(3)
        rows = []
        for E, n, k in ((8, 14336, 4096), (32, 4096, 4096), (64, 2048, 7168), (128, 1536, 4096)):
            W = [torch.randint(0, 256, (E, n, k // 2), dtype=torch.uint8, generator=g).to(dev) for _ in range(3)]
            WS = [torch.randint(120, 135, (E, n, k // 32), dtype=torch.uint8, generator=g).to(dev) for _ in range(3)]
            for per_e in (1, 16, 32, 64, 128, 192):
                if E * per_e > 8192:
                    continue
                total = E * per_e
                x = torch.randint(0, 256, (total, k // 2), dtype=torch.uint8, generator=g).to(dev)
                xs = torch.randint(120, 135, (total, k // 32), dtype=torch.uint8, generator=g).to(dev)
                out = torch.empty(total, n, dtype=torch.bfloat16, device=dev)
                for ragged in (False, True):
                    cnt = (np.random.default_rng(per_e).multinomial(total, np.ones(E) / E) if ragged
                           else np.full(E, per_e))
                    off = torch.tensor(np.concatenate([[0], np.cumsum(cnt)]), dtype=torch.int32, device=dev)
                    us = {}
                    # (the library's choice first and last, the shorter time kept, as in decode_sweep)
                    for name, v in (("auto", L.VARIANT_AUTO), ("mid", L.VARIANT_MID_M),
                                    ("t128x128", L.VARIANT_T128x128_W2x2), ("t256x256", L.VARIANT_T256x256_W4x2),
                                    ("auto", L.VARIANT_AUTO)):
                        state = {"i": 0}

                        def run(count):
                            for _ in range(count):
                                i = state["i"] % 3
                                state["i"] += 1
                                wave_amd.mxfp4_gemm_grouped(x, xs, W[i], WS[i], off, out, variant=v)

                        _, per, _ = timed(torch, run, min(args.steps, 60), 10)
                        us[name] = min(us.get(name, 1e9), round(per * 1e6, 1))
                    used = int((cnt > 0).sum())  # an expert without rows is not read
                    nbytes = used * n * (k // 2 + k // 32) + total * (k // 2 + k // 32) + total * n * 2
                    rows.append({"experts": E, "n": n, "k": k, "rows_per_expert": per_e,
                                 "groups": "multinomial" if ragged else "even", "us": us, "bytes": nbytes,
                                 "auto_frac_of_hbm_peak": round(nbytes / (us["auto"] * 1e-6) / 1e9 / PEAK_HBM_GBPS, 4)})
                del x, xs, out
            del W, WS
        worst = max(r["us"]["auto"] / min(r["us"].values()) for r in rows)
        print(json.dumps(dict(common, **{
            "metric": "grouped MXFP4 GEMM at serving batches: worst ratio of the library's choice to the best kernel",
            "value": round(worst, 3), "unit": "x", "higher_is_better": False,
            "ms_per_step": round(sum(r["us"]["auto"] for r in rows) * 1e-3, 3),
            "dtype": "mxfp4 (e2m1 x e8m0) in, f32 accumulate, bf16 out",
            "data": "synthetic (seeded uniform), weights from HBM",
            "config": {"workload": f"moe_serving: {len(rows)} (experts, N, K, rows per expert, even or multinomial groups)"},
            "shapes": rows})))
        return

    if args.workload == "ref_shapes":
        # every (M, N) of the reference's benchmark list at its K = 16000 (a partial last K tile), bf16 out
        import math

        k = REF_SHAPES_K
        rows = []
        first = True
        for m in sorted(REF_SHAPES_MN):
            for n in REF_SHAPES_MN[m]:
                sets = make_gpu_inputs(torch, m, n, k, 1, (124, 130), dev, copies=1)
                out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
                flops = gemm_flops(m, n, k)
                steps = max(10, min(args.steps, int(0.05 / (flops / 4.0e15))))
                if not first:   # the clocks are up after the first shape: a short settle keeps them there
                    SETTLE["ms"] = 10.0
                first = False
                _, per, _ = time_gemm(torch, wave_amd, sets, out, steps, max(5, steps // 3), variant=args.variant)
                rows.append((m, n, per, flops / per / 1e12))
                del sets, out
        geo = math.exp(sum(math.log(r[3]) for r in rows) / len(rows))
        big = [r for r in rows if r[0] * r[1] >= 4096 * 4096]
        geo_big = math.exp(sum(math.log(r[3]) for r in big) / len(big))
        print(json.dumps(dict(common, **{
            "metric": "MXFP4 GEMM TFLOPS over the reference's benchmark shapes (K = 16000), geometric mean",
            "value": round(geo, 1), "unit": "TFLOP/s",
            "ms_per_step": round(sum(r[2] for r in rows) * 1e3, 3),
            "dtype": "mxfp4 (e2m1 x e8m0) in, f32 accumulate, bf16 out",
            "data": "synthetic (seeded uniform nibbles and scales)",
            "config": {"workload": f"ref_shapes: {len(rows)} (M, N) pairs, K = {k}, bf16 out, seed 1"},
            "geomean_tflops_mn_ge_4096x4096": round(geo_big, 1),
            "shapes": [{"m": r[0], "n": r[1], "us": round(r[2] * 1e6, 1), "tflops": round(r[3], 1)} for r in rows]})))
        return

    if args.workload == "moe_glue":
        # the steps around cfg4: 4096 tokens x top-2 of 8 experts, hidden 4096, intermediate 14336, bf16
        tokens, topk, E, hidden, inter = 4096, 2, 8, 4096, 14336
        g = torch.Generator(device=dev).manual_seed(3)
        ids = torch.stack([torch.randperm(E, device=dev, generator=g)[:topk] for _ in range(tokens)]).to(torch.int32)
        n_ent = tokens * topk
        sorted_ids = torch.empty(n_ent, dtype=torch.int32, device=dev)
        expert_ids = torch.empty(n_ent, dtype=torch.int32, device=dev)
        total = torch.empty(1, dtype=torch.int32, device=dev)
        offs = torch.empty(E + 1, dtype=torch.int32, device=dev)
        acts = [torch.randn(tokens, hidden, device=dev, generator=g).to(torch.bfloat16) for _ in range(3)]
        gemm1 = [torch.randn(n_ent, 2 * inter, device=dev, generator=g).to(torch.bfloat16) for _ in range(2)]

        def timed_fn(fn):
            state = {"i": 0}

            def run(count):
                for _ in range(count):
                    fn(state["i"])
                    state["i"] += 1

            return timed(torch, run, args.steps, args.warmup)[1]

        # straight through the C ABI with outputs allocated once: the kernels are shorter than a Python wrapper call
        lib, st = _lib.load(), torch.cuda.current_stream().cuda_stream
        q1 = torch.empty(n_ent, hidden // 2, dtype=torch.uint8, device=dev)
        s1 = torch.empty(n_ent, hidden // 32, dtype=torch.uint8, device=dev)
        q2 = torch.empty(n_ent, inter // 2, dtype=torch.uint8, device=dev)
        s2 = torch.empty(n_ent, inter // 32, dtype=torch.uint8, device=dev)
        t_align = timed_fn(lambda i: lib.wave_mxfp4_moe_align_block_size(
            ids.data_ptr(), 0, n_ent, E, 1, sorted_ids.data_ptr(), n_ent, expert_ids.data_ptr(), n_ent,
            total.data_ptr(), offs.data_ptr(), st))
        t_gather = timed_fn(lambda i: lib.wave_mxfp4_quantize_rows(
            acts[i % 3].data_ptr(), _lib.IN_BF16, tokens, sorted_ids.data_ptr(), topk, q1.data_ptr(), s1.data_ptr(),
            n_ent, hidden, _lib.SCALE_ROW_MAJOR, st))
        t_act = timed_fn(lambda i: lib.wave_mxfp4_silu_and_mul_quantize(
            gemm1[i % 2].data_ptr(), gemm1[i % 2].data_ptr() + 2 * inter, 2 * inter, 2 * inter, _lib.IN_BF16,
            q2.data_ptr(), s2.data_ptr(), n_ent, inter, _lib.SCALE_ROW_MAJOR, st))
        b_gather = n_ent * hidden * 2 + n_ent * hidden // 2 + n_ent * hidden // 32   # every source row is read top_k times
        b_act = n_ent * inter * 4 + n_ent * inter // 2 + n_ent * inter // 32
        gbps = b_act / t_act / 1e9
        print(json.dumps(dict(common, **{
            "metric": "MoE glue: gated activation + quantiser GB/s % HBM", "value": round(gbps, 1), "unit": "GB/s",
            "ms_per_step": round(t_act * 1e3, 4), "dtype": "bf16 in, e2m1 + e8m0 out", "data": "synthetic (normal)",
            "config": {"workload": f"moe_glue: {tokens} tokens x top-{topk} of {E} experts, hidden {hidden}, "
                                   f"intermediate {inter}"},
            "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                         "frac": round(gbps / PEAK_HBM_GBPS, 4), "traffic": None,
                         "kernel": "quantize_kernel (gated)", "launch_us": round(t_act * 1e6, 2)},
            "moe_align_block_size_us": round(t_align * 1e6, 2),
            "gathered_quantiser": {"launch_us": round(t_gather * 1e6, 2), "gbps": round(b_gather / t_gather / 1e9, 1),
                                   "bytes": b_gather}})))
        return

    if args.workload == "moe_layer":
        leg = leg_moe_layer(torch, wave_amd, dev, args.steps, args.warmup, tokens=args.moe_tokens)
        print(json.dumps(dict(common, **{
            "metric": "MoE expert MLP (align, gather + quantise, grouped GEMM + gated quantiser, grouped GEMM) TFLOPS",
            "value": leg["tflops"], "unit": "TFLOP/s", "ms_per_step": round(leg["layer_us"] * 1e-3, 4),
            "dtype": "bf16 activations, mxfp4 operands, f32 accumulate, bf16 out", "data": "synthetic (normal activations, uniform weights)",
            "config": {"workload": leg["workload"]},
            # a serving batch (the rows per expert the grouped calls give to the mid-M kernel) reads every weight for
            # a handful of rows: the layer is priced against HBM; a prefill batch against the MFMA peak
            "roofline": ({"bound": "hbm", "achieved": round(leg["algorithmic_bytes"] / leg["layer_us"] / 1e3, 1),
                          "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                          "frac": round(leg["algorithmic_bytes"] / leg["layer_us"] / 1e3 / PEAK_HBM_GBPS, 4), "traffic": None,
                          "kernel": "mid_gemm_kernel (grouped), all steps of the layer", "launch_us": leg["layer_us"]}
                         if leg["rows_per_expert"] <= 160 else
                         {"bound": "mfma", "achieved": leg["tflops"], "peak": PEAK_MXFP4_TFLOPS, "unit": "TFLOP/s",
                          "frac": leg["frac_of_mxfp4_peak"], "traffic": None, "kernel": "persist_gemm_kernel (grouped)",
                          "launch_us": leg["layer_us"]}),
            "steps_us": leg["steps_us"], "sum_of_steps_us": leg["sum_of_steps_us"],
            "separate_activation_kernel": leg["separate_activation_kernel"]})))
        return

    if args.workload == "cfg4":
        leg = leg_cfg4(torch, wave_amd, dev, args.steps, args.warmup, args.variant)
        print(json.dumps(dict(common, **{
            "metric": "grouped (MoE) MXFP4 GEMM TFLOPS", "value": leg["tflops"], "unit": "TFLOP/s",
            "ms_per_step": round(leg.pop("wall_s_per_step") * 1e3, 4),
            "dtype": "mxfp4 (e2m1 x e8m0) in, f32 accumulate, bf16 out", "data": "synthetic (seeded uniform)",
            "config": {"workload": leg["workload"], "variant": args.variant}, "settle_ms": leg["settle_ms"],
            "roofline": {"bound": "mfma", "achieved": leg["tflops"], "peak": PEAK_MXFP4_TFLOPS, "unit": "TFLOP/s",
                         "frac": leg["frac_of_mxfp4_peak"], "traffic": read_traffic("cfg4"), "kernel": leg["kernel"],
                         "launch_us": leg["launch_us"]},
            "resident_weight_scales": leg["resident_weight_scales"], "serving_batch": leg["serving_batch"]})))
        return

    if args.workload == "mxfp8":
        leg = leg_mxfp8(torch, wave_amd, dev, args.steps, args.warmup, args.variant)
        print(json.dumps(dict(common, **{
            "metric": "MXFP8 GEMM TFLOPS + % of FP8 MFMA peak (8192^3)", "value": leg["tflops"], "unit": "TFLOP/s",
            "ms_per_step": round(leg.pop("wall_s_per_step") * 1e3, 4),
            "dtype": "mxfp8 (e5m2 x e8m0) in, f32 accumulate, f32 out", "data": "synthetic (normal values, seeded)",
            "config": {"workload": leg["workload"], "variant": args.variant}, "settle_ms": leg["settle_ms"],
            "e5m2_x_e2m1": leg["e5m2_x_e2m1"], "b_preshuffled": leg["b_preshuffled"],
            "roofline": {"bound": "mfma", "achieved": leg["tflops"], "peak": PEAK_MXFP8_TFLOPS, "unit": "TFLOP/s",
                         "frac": leg["frac_of_mxfp8_peak"], "traffic": read_traffic("mxfp8"), "kernel": leg["kernel"],
                         "launch_us": leg["launch_us"]}})))
        return

    m, n, k, od, seed, srange = WORKLOADS[args.workload]
    out_dtype = torch.bfloat16 if od == "bf16" else torch.float32
    out_bytes = 2 if od == "bf16" else 4
    memory_bound = m <= 128
    # memory-bound shapes rotate distinct operand sets so B is not cache resident
    copies = 4 if memory_bound else 1
    sets = make_gpu_inputs(torch, m, n, k, seed, srange, dev, copies=copies)
    out = torch.empty(m, n, dtype=out_dtype, device=dev)
    wall, per_launch, settle_ms = time_gemm(torch, wave_amd, sets, out, args.steps, args.warmup, variant=args.variant)

    # HBM bytes per launch of the dominant kernel: rocprofv3 FETCH_SIZE + WRITE_SIZE runs of this command, scaled
    # by a device copy of known size, kept in profiles/hbm_traffic.txt (not measurable from here); None without a line
    measured_traffic = read_traffic(args.workload) if args.variant == 0 else None
    flops, nbytes = gemm_flops(m, n, k), gemm_bytes(m, n, k, out_bytes)
    ms_per_step = wall / args.steps * 1e3
    tflops = flops / (wall / args.steps) / 1e12
    if memory_bound:
        achieved = nbytes / per_launch / 1e9
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                    "frac": round(achieved / PEAK_HBM_GBPS, 4), "traffic": measured_traffic,
                    "kernel": "stream_gemm_kernel" if m <= 16 else "mid_gemm_kernel",
                    "launch_us": round(per_launch * 1e6, 2)}
    else:
        achieved = flops / per_launch / 1e12
        roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_MXFP4_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(achieved / PEAK_MXFP4_TFLOPS, 4), "traffic": measured_traffic,
                    "kernel": "persist_gemm_kernel" if (n % 256 == 0 and ((m + 255) // 256) * (n // 256) > 256) else "tile_gemm_kernel",
                    "launch_us": round(per_launch * 1e6, 2)}

    result = dict(common, **{
        "metric": "MXFP4 GEMM TFLOPS + % of FP4 MFMA peak (8192^3); GB/s % HBM at M=16",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "ms_per_step": round(ms_per_step, 4),
        "settle_ms": round(settle_ms, 1),
        "dtype": "mxfp4 (e2m1 x e8m0) in, f32 accumulate, " + od + " out",
        "data": "synthetic (seeded uniform nibbles and scales), random weights",
        "config": {"workload": f"{args.workload}: M={m} N={n} K={k} {od} out seed {seed}",
                   "variant": args.variant, "operand_sets_rotated": copies},
        "frac_of_mxfp4_peak": round(tflops / PEAK_MXFP4_TFLOPS, 4),
        "gbps": round(nbytes / (wall / args.steps) / 1e9, 1),
        "roofline": roofline,
    })

    if not memory_bound and args.variant == 0:
        # The same launch with both scale tensors handed over in the MFMA operand order (the reference's headline
        # kernels take scales preshuffled ahead of the timed region the same way, examples/python/7.1_schedule.py
        # :323-375; a quantiser can write that order directly): no re-layout pass in front of the GEMM.
        from wave_amd import _lib as L
        x, xs, w, ws = sets[0]
        xs32 = wave_amd.scale_convert(xs, m, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32)
        ws32 = wave_amd.scale_convert(ws, n, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32)
        _, pper, _ = time_gemm(torch, wave_amd, [(x, xs32, w, ws32)], out, args.steps, args.warmup,
                               a_scale_layout=L.SCALE_MFMA32, b_scale_layout=L.SCALE_MFMA32)
        result["preshuffled_scales"] = {
            "workload": "the same operands, scales already in MFMA operand order (no re-layout launch)",
            "launch_us": round(pper * 1e6, 2), "tflops": round(flops / pper / 1e12, 1),
            "frac_of_mxfp4_peak": round(flops / pper / 1e12 / PEAK_MXFP4_TFLOPS, 4),
        }
        # ... and in e8m0_shuffle order, the format the reference's preshuffled-scale kernels take
        # (wave_lang/kernel/wave/utils/mxfp_utils.py:113-128): read in place by the persistent kernels
        xsh = wave_amd.scale_convert(xs, m, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_E8M0_SHUFFLE)
        wsh = wave_amd.scale_convert(ws, n, k // 32, L.SCALE_ROW_MAJOR, L.SCALE_E8M0_SHUFFLE)
        _, sper, _ = time_gemm(torch, wave_amd, [(x, xsh, w, wsh)], out, args.steps, args.warmup,
                               a_scale_layout=L.SCALE_E8M0_SHUFFLE, b_scale_layout=L.SCALE_E8M0_SHUFFLE)
        _, iper, _ = time_gemm(torch, wave_amd, [(x, xsh, w, wsh)], out, args.steps, args.warmup, workspace=False,
                               a_scale_layout=L.SCALE_E8M0_SHUFFLE, b_scale_layout=L.SCALE_E8M0_SHUFFLE)
        result["e8m0_shuffled_scales"] = {
            "workload": "the same operands, scales in the reference's e8m0_shuffle order: with scratch (re-laid by one "
                        "launch, the library's choice), and without (read in place by the persistent kernel)",
            "launch_us": round(sper * 1e6, 2), "tflops": round(flops / sper / 1e12, 1),
            "frac_of_mxfp4_peak": round(flops / sper / 1e12 / PEAK_MXFP4_TFLOPS, 4),
            "in_place_no_scratch_us": round(iper * 1e6, 2),
        }
        del xsh, wsh
        # roofline: the dominant kernel by itself, i.e. this leg's launches (a call with row-major scales is that
        # kernel + the scale re-layout launch in front of it: `call_us`, the figure `value` is computed from)
        roofline["call_us"] = roofline["launch_us"]
        roofline["launch_us"] = round(pper * 1e6, 2)
        roofline["achieved"] = round(flops / pper / 1e12, 1)
        roofline["frac"] = round(flops / pper / 1e12 / PEAK_MXFP4_TFLOPS, 4)
        if n % 256 == 0 and k % 512 == 0 and k >= 1536:
            # ... and B in b_preshuffle order on top (static weights, preshuffled once, as the reference's
            # asymmetric kernels assume: templates/tagged_mxfp4_gemm.py:950-991): A through LDS, B straight from
            # global memory into registers
            wp = wave_amd.b_preshuffle(w)
            _, bper, _ = time_gemm(torch, wave_amd, [(x, xs32, wp, ws32)], out, args.steps, args.warmup,
                                   a_scale_layout=L.SCALE_MFMA32, b_scale_layout=L.SCALE_MFMA32, b_layout=L.B_PRESHUFFLE)
            result["preshuffled_b"] = {
                "workload": "the same operands, B in b_preshuffle order and scales in MFMA operand order",
                "kernel": "asym_gemm_kernel", "launch_us": round(bper * 1e6, 2), "tflops": round(flops / bper / 1e12, 1),
                "frac_of_mxfp4_peak": round(flops / bper / 1e12 / PEAK_MXFP4_TFLOPS, 4),
            }
            del wp
        if args.workload == "cfg2" and not args.no_legs:
            # What this chip, in this run, lets the matrix pipes do: the scaled FP4 MFMA alone (no memory traffic,
            # wave_amd/csrc/mfma_probe.hip) on random and on all-zero operand bytes, and the headline kernel on
            # all-zero operands (same instruction stream and traffic as on the seeded data, less power per
            # instruction).  On random bytes the chip is power-limited well below its 2.4 GHz peak clock, so
            # `frac_of_mfma_alone` is the headline kernel against the ceiling measured beside it, `frac` against
            # the published peak.
            rows, _ = mfma_ceiling(torch, dev, args.steps, args.warmup, compact=True)
            by = {r["operands"]: r for r in rows}
            zx, zw = torch.zeros_like(x), torch.zeros_like(w)
            _, zper, _ = time_gemm(torch, wave_amd, [(zx, xs32, zw, ws32)], out, args.steps, args.warmup,
                                   a_scale_layout=L.SCALE_MFMA32, b_scale_layout=L.SCALE_MFMA32)
            del zx, zw
            result["power_ceiling"] = {
                "workload": "v_mfma_scale_f32_32x32x64_f8f6f4 alone, 8 waves per CU, 8000 x 32 per wave and launch, on "
                            "uniformly random bytes and on zeros; the headline kernel on all-zero A and B",
                "mfma_random_tflops": by["random"]["tflops"], "mfma_random_clock_ghz": by["random"]["mfma_clock_ghz"],
                "mfma_zero_tflops": by["zeros"]["tflops"], "mfma_zero_clock_ghz": by["zeros"]["mfma_clock_ghz"],
                "gemm_zero_us": round(zper * 1e6, 2), "gemm_zero_tflops": round(flops / zper / 1e12, 1),
                "gemm_zero_frac_of_mfma_zero": round(flops / zper / 1e12 / by["zeros"]["tflops"], 4),
            }
            roofline["frac_of_mfma_alone"] = round(roofline["achieved"] / by["random"]["tflops"], 4)
        del xs32, ws32
    del sets, out

    if not args.no_legs and args.workload == "cfg2":
        # the decode shapes of the metric's second half: M = 16 (its target), and M = 1, 32, 64 and 128 beside it
        for name in ("cfg3_m16", "cfg3_m1", "cfg3_m32", "cfg3_m64", "cfg3_m128", "cfg3_m256"):
            dm, dn, dk, _, dseed, drange = WORKLOADS[name]
            dsets = make_gpu_inputs(torch, dm, dn, dk, dseed, drange, dev, copies=4)
            dout = torch.empty(dm, dn, dtype=torch.bfloat16, device=dev)
            dsteps = max(args.steps, 20) * (4 if name == "cfg3_m16" else 1)
            _, dper, dsettle = time_gemm(torch, wave_amd, dsets, dout, dsteps, args.warmup)
            dbytes = gemm_bytes(dm, dn, dk, 2)
            result["decode_m%d" % dm] = {
                "workload": f"{name}: M={dm} N={dn} K={dk} bf16 out seed {dseed}, 4 operand sets rotated (HBM-cold B)",
                "launch_us": round(dper * 1e6, 2),
                "gbps": round(dbytes / dper / 1e9, 1),
                "frac_of_hbm_peak": round(dbytes / dper / 1e9 / PEAK_HBM_GBPS, 4),
                "bytes": dbytes, "steps": dsteps, "settle_ms": round(dsettle, 1),
                "kernel": "stream_gemm_kernel" if dm <= 16 else "mid_gemm_kernel",
                "traffic": read_traffic(name),
            }
            if dm > 16:
                # resident weights: B's scales converted once to the MFMA operand order (wave_mxfp4_scale_convert),
                # as a serving stack would keep them; A's scales stay row-major
                from wave_amd import _lib as L
                rsets = [(x, xs, w, wave_amd.scale_convert(ws, dn, dk // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32))
                         for (x, xs, w, ws) in dsets]
                _, rper, _ = time_gemm(torch, wave_amd, rsets, dout, dsteps, args.warmup, b_scale_layout=L.SCALE_MFMA32)
                result["decode_m%d" % dm]["resident_weight_scales"] = {
                    "workload": "the same call with B's scales already in MFMA operand order",
                    "launch_us": round(rper * 1e6, 2), "gbps": round(dbytes / rper / 1e9, 1),
                    "frac_of_hbm_peak": round(dbytes / rper / 1e9 / PEAK_HBM_GBPS, 4)}
                if dm > 128:
                    # ... and B in b_preshuffle order on top (static weights, preshuffled once, as the reference's
                    # asymmetric kernels assume), A's scales in MFMA order as the quantiser writes them: A through
                    # LDS, B straight from global memory into registers
                    psets = [(x, wave_amd.scale_convert(xs, dm, dk // 32, L.SCALE_ROW_MAJOR, L.SCALE_MFMA32),
                              wave_amd.b_preshuffle(w), ws32) for (x, xs, w, ws32) in rsets]
                    _, pper, _ = time_gemm(torch, wave_amd, psets, dout, dsteps, args.warmup, a_scale_layout=L.SCALE_MFMA32,
                                           b_scale_layout=L.SCALE_MFMA32, b_layout=L.B_PRESHUFFLE)
                    result["decode_m%d" % dm]["preshuffled_b"] = {
                        "workload": "the same operands, B in b_preshuffle order and both scale tensors in MFMA operand order",
                        "kernel": "midb_gemm_kernel", "launch_us": round(pper * 1e6, 2),
                        "gbps": round(dbytes / pper / 1e9, 1),
                        "frac_of_hbm_peak": round(dbytes / pper / 1e9 / PEAK_HBM_GBPS, 4)}
                    del psets
                del rsets
            del dsets, dout

        # the step in front of the GEMM: quantise the bf16 activation of this workload
        qper, qbytes, qsettle = time_quantize(torch, wave_amd, m, k, args.steps, args.warmup, dev)
        result["quantize_a"] = {
            "workload": f"bf16 [{m}, {k}] -> e2m1 + e8m0 (e8m0_shuffle order), 3 inputs rotated",
            "kernel": "quantize_kernel",
            "launch_us": round(qper * 1e6, 2),
            "gbps": round(qbytes / qper / 1e9, 1),
            "frac_of_hbm_peak": round(qbytes / qper / 1e9 / PEAK_HBM_GBPS, 4),
            "bytes": qbytes, "settle_ms": round(qsettle, 1),
        }
        # the other configurations and the 8-bit operands, each with its own settle load
        leg = leg_cfg4(torch, wave_amd, dev, args.steps, args.warmup)
        leg.pop("wall_s_per_step")
        result["cfg4_grouped"] = leg
        result["cfg5"] = leg_dense(torch, wave_amd, dev, "cfg5", args.steps, args.warmup)
        leg = leg_mxfp8(torch, wave_amd, dev, args.steps, args.warmup)
        leg.pop("wall_s_per_step")
        result["mxfp8"] = leg
        torch.cuda.empty_cache()
        result["moe_layer"] = leg_moe_layer(torch, wave_amd, dev, min(args.steps, 50), min(args.warmup, 20))
        torch.cuda.empty_cache()
        # the same layer at a serving batch (16 rows per expert): every weight read once for a handful of rows, the
        # layer priced against HBM (frac_of_hbm_peak)
        result["moe_layer_serving"] = leg_moe_layer(torch, wave_amd, dev, args.steps, args.warmup, tokens=64)

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, m, n, k, seed, srange, args.cpu_rows)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
