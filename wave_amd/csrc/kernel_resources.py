"""Registers, scratch, LDS and occupancy of every kernel of libwave_mxfp4.so.

The Makefile compiles with ``-Rpass-analysis=kernel-resource-usage`` and keeps the
compiler's remarks beside each object (``<object>.remarks``).  This module parses
them; run as a script it prints one line per kernel:

    python wave_amd/csrc/kernel_resources.py [--hot]

The reference gates its generated kernels on the same figures (VGPR count,
instruction count, MFMA density: wave_lang/kernel/wave/perf/
bench_mxfp4_comparison.py:948-1016).  A kernel of the hot paths that needs
scratch memory would reload registers inside its main loop, and every reload
waits for the whole memory queue; tests/test_kernel_resources.py fails if one does.
"""

import glob
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))

FIELDS = {
    "TotalSGPRs": "sgpr",
    "VGPRs": "vgpr",
    "AGPRs": "agpr",
    "ScratchSize [bytes/lane]": "scratch",
    "Occupancy [waves/SIMD]": "occupancy",
    "SGPRs Spill": "sgpr_spill",
    "VGPRs Spill": "vgpr_spill",
    "LDS Size [bytes/block]": "static_lds",
}

# kernels whose main loops the throughput figures depend on
HOT = ("persist_gemm_kernel", "persist_gemm_gated_kernel", "persist_gemm_fp8_kernel", "asym_gemm_kernel", "asym8_gemm_kernel", "tile_gemm_kernel", "stream_gemm_kernel", "mid_gemm_kernel", "midb_gemm_kernel",
       "quantize_kernel")


def _demangle(names):
    tool = "/opt/rocm/llvm/bin/llvm-cxxfilt"
    if not os.path.exists(tool):
        tool = "c++filt"
    try:
        out = subprocess.run([tool], input="\n".join(names), capture_output=True, text=True, check=True).stdout
        return out.splitlines()
    except (OSError, subprocess.CalledProcessError):
        return list(names)


def parse(directory=HERE):
    """[{name, mangled, file, sgpr, vgpr, agpr, scratch, occupancy, ...}] over all <object>.remarks files."""
    kernels = []
    for path in sorted(glob.glob(os.path.join(directory, "*.o.remarks"))):
        cur = None
        with open(path) as fh:
            for line in fh:
                m = re.search(r"remark:\s+(.*?): (\S+) \[-Rpass-analysis", line)
                if not m:
                    continue
                key, val = m.group(1).strip(), m.group(2)
                if key == "Function Name":
                    cur = {"mangled": val, "file": os.path.basename(path)[: -len(".o.remarks")] + ".hip"}
                    kernels.append(cur)
                elif cur is not None and key in FIELDS:
                    cur[FIELDS[key]] = int(val)
    for k, name in zip(kernels, _demangle([k["mangled"] for k in kernels])):
        k["name"] = re.sub(r"^void |wave_mxfp4::|\(wave_mxfp4::GemmParams\)|\(anonymous namespace\)::", "", name)
    return kernels


def is_hot(kernel):
    return any(h in kernel["name"] for h in HOT)


def main():
    hot_only = "--hot" in sys.argv[1:]
    rows = [k for k in parse() if not hot_only or is_hot(k)]
    if not rows:
        print("no <object>.remarks files: build the library first (make -C wave_amd/csrc)", file=sys.stderr)
        return 1
    print(f"{'VGPR':>5} {'AGPR':>5} {'SGPR':>5} {'scratch':>8} {'occ':>4} {'sgpr->vgpr':>10}  kernel")
    for k in rows:
        print(f"{k.get('vgpr', -1):5d} {k.get('agpr', -1):5d} {k.get('sgpr', -1):5d} {k.get('scratch', -1):8d} "
              f"{k.get('occupancy', -1):4d} {k.get('sgpr_spill', -1):10d}  {k['name']}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
