"""Kernel resource gate (CPU only): the compiler's own report of registers and
scratch memory for every kernel of the library, read from the remarks the build
keeps beside each object.

The reference gates its generated MXFP4 kernels on VGPR count, instruction count
and MFMA density against a baseline
(wave_lang/kernel/wave/perf/bench_mxfp4_comparison.py:948-1016).  Here the gate
is the one that matters for hand-scheduled loops with counted waits: no kernel of
a hot path may need scratch memory (a register reloaded inside the main loop
waits for the whole memory queue), and the register budget must keep the
occupancy its launch assumes.
"""

import os
import subprocess

import pytest

from wave_amd.csrc import kernel_resources as kr

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "wave_amd", "csrc")

# Kernels that do use scratch, with the most they may use (bytes per lane).  The first two are not on a path the
# library picks by itself for the shapes the throughput figures are quoted on:
#  * the 4-wave one-tile-per-workgroup 256x256 kernel (variant T256x256_W2x2; AUTO takes the 8-wave one),
#  * the streaming kernel's 49..64-row instantiation with one or two waves along K (all 512 registers hold A).
#  * the B-direct kernels with bf16 output: a handful of registers are spilled and reloaded once per OUTPUT TILE,
#    around the accumulator read-out between two K loops (5 stores + 5 loads per 4096 MFMAs of a wave), none
#    inside a K loop.
KNOWN_SCRATCH = {
    "asym_gemm_kernel<true, false>": 32,
    "asym8_gemm_kernel<true,": 32,
    "tile_gemm_kernel<TileCfg<256, 256, 2, 2>": 160,
    "stream_gemm_kernel<4, true, 1>": 32,
    "stream_gemm_kernel<4, true, 2>": 32,
}


@pytest.fixture(scope="module")
def kernels():
    # The remarks are build output (not tracked): make brings every object, and with it its remarks file, up to
    # date with its source and the common headers (a no-op when they are; about a minute from scratch).  A remarks
    # file that is missing although its object is current (objects built by something else than the Makefile)
    # forces a full rebuild.
    subprocess.check_call(["make", "-C", CSRC, "-j8", "libwave_mxfp4.so"], stdout=subprocess.DEVNULL)
    srcs = [f for f in os.listdir(CSRC) if f.startswith("mxfp4_") and f.endswith(".hip")]
    ks = kr.parse(CSRC)
    if not ks or any(not os.path.exists(os.path.join(CSRC, f[:-4] + ".o.remarks")) for f in srcs):
        subprocess.check_call(["make", "-C", CSRC, "-B", "-j8", "libwave_mxfp4.so"], stdout=subprocess.DEVNULL)
        ks = kr.parse(CSRC)
    assert ks, "no kernel-resource remarks beside the objects"
    return ks


def test_every_hot_kernel_family_is_reported(kernels):
    names = " ".join(k["name"] for k in kernels)
    for family in ("persist_gemm_kernel", "tile_gemm_kernel", "stream_gemm_kernel", "quantize_kernel",
                   "splitk_reduce_kernel", "naive_gemm_kernel"):
        assert family in names, family


def test_hot_kernels_use_no_scratch(kernels):
    hot = [k for k in kernels if kr.is_hot(k)]
    assert len(hot) >= 40
    bad = []
    for k in hot:
        allowed = max([v for pre, v in KNOWN_SCRATCH.items() if k["name"].startswith(pre)], default=0)
        if k["scratch"] > allowed or k["vgpr_spill"] > 0 and allowed == 0:
            bad.append((k["name"], k["scratch"], k["vgpr_spill"]))
    assert not bad, bad


def test_register_budget_matches_launch_assumptions(kernels):
    by_name = {k["name"]: k for k in kernels}
    for name, k in by_name.items():
        assert k["vgpr"] + k["agpr"] <= 512, name
        # the persistent 8-wave kernels run two waves per SIMD (one workgroup of 8 waves per CU)
        if name.startswith("persist_gemm_kernel<TileCfg<256, 256, 4, 2>"):
            assert k["occupancy"] >= 2 and k["scratch"] == 0, (name, k)
        # the quantiser is a bandwidth kernel: it must stay at full occupancy
        if name.startswith("quantize_kernel"):
            assert k["occupancy"] == 8, (name, k)
        # the mid-M kernel's shallow configuration is launched so that two workgroups of five waves share a CU:
        # three waves on some SIMD
        if name.startswith("mid_gemm_kernel<MidCfg<32, true, true>") or name.startswith("mid_gemm_kernel<MidCfg<32, false, true>"):
            assert k["occupancy"] >= 3 and k["scratch"] == 0, (name, k)


def test_summary_script_runs():
    out = subprocess.run(["python", os.path.join(CSRC, "kernel_resources.py"), "--hot"], capture_output=True, text=True)
    assert out.returncode == 0 and "persist_gemm_kernel" in out.stdout
