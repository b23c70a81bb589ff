"""ctypes binding of ``csrc/libwave_mxfp4.so`` (the C ABI declared in
``include/wave_mxfp4.h``).  There is no fallback: if the library is missing or
does not load, every operator of this package raises."""

from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# WAVE_MXFP4_LIB points at another build of the same ABI (e.g. an experiment)
LIB_PATH = os.environ.get("WAVE_MXFP4_LIB") or os.path.join(_HERE, "csrc", "libwave_mxfp4.so")

ABI_VERSION = 10

# status codes of include/wave_mxfp4.h
OK = 0
ERR_NULL_POINTER = -1
ERR_BAD_SHAPE = -2
ERR_BAD_ENUM = -3
ERR_MISALIGNED = -4
ERR_WORKSPACE = -5
ERR_BAD_SPLIT = -6
ERR_HIP = -7
ERR_UNSUPPORTED = -8

OUT_F32, OUT_BF16 = 0, 1
SCALE_ROW_MAJOR, SCALE_E8M0_SHUFFLE, SCALE_MFMA32, SCALE_PER_ROW = 0, 1, 2, 3
B_ROW_MAJOR, B_PRESHUFFLE = 0, 1
IN_F32, IN_BF16, IN_F16 = 0, 1, 2
MXFP8_E4M3, MXFP8_E5M2, MXFP8_B_E2M1 = 0, 1, 2
MXFP8_E2M1 = MXFP8_B_E2M1  # one operand (x or w_t, not both) packed MXFP4 against an 8-bit other

VARIANT_AUTO = 0
VARIANT_T256x256_W2x2 = 1
VARIANT_T256x256_W4x2 = 2
VARIANT_T128x128_W2x2 = 3
VARIANT_SKINNY = 4
VARIANT_NAIVE = 5
VARIANT_T128x256_W2x2 = 6
VARIANT_T256x256_W1x4_BDIRECT = 7
VARIANT_MID_M = 8
VARIANT_T256x192_W4x2 = 9
VARIANT_MID_M_BDIRECT = 10

# every symbol include/wave_mxfp4.h declares
EXPORTS = (
    "wave_mxfp4_gemm",
    "wave_mxfp4_workspace_bytes",
    "wave_mxfp4_gemm_static",
    "wave_mxfp4_static_scratch_bytes",
    "wave_mxfp4_gemm_grouped",
    "wave_mxfp4_grouped_workspace_bytes",
    "wave_mxfp8_gemm",
    "wave_mxfp8_workspace_bytes",
    "wave_mxfp8_b_preshuffle",
    "wave_mxfp8_gemm_b_preshuffled",
    "wave_mxfp4_to_f32",
    "wave_mxfp4_e8m0_to_f32",
    "wave_mxfp4_dequant",
    "wave_mxfp4_e8m0_shuffle",
    "wave_mxfp4_e8m0_shuffle_bytes",
    "wave_mxfp4_scale_convert",
    "wave_mxfp4_b_preshuffle",
    "wave_mxfp4_quantize",
    "wave_mxfp4_quantize_rows",
    "wave_mxfp4_moe_align_block_size",
    "wave_mxfp4_silu_and_mul",
    "wave_mxfp4_silu_and_mul_quantize",
    "wave_mxfp4_gemm_gated_quantize",
    "wave_mxfp4_interleave_gate_up",
    "wave_mxfp4_status_string",
    "wave_mxfp4_last_hip_error",
    "wave_mxfp4_abi_version",
)

_lib = None


def load():
    """Load the shared library once and declare its prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.dirname(LIB_PATH)}` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no CPU fallback")
    lib = ctypes.CDLL(LIB_PATH)
    p, i64, i32, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
    lib.wave_mxfp4_gemm.argtypes = [p, p, p, p, p, i64, i64, i64, i32, i32, i32, i32, i32, p, sz, i32, p]
    lib.wave_mxfp4_gemm.restype = i32
    lib.wave_mxfp4_workspace_bytes.argtypes = [i64, i64, i64, i32, i32]
    lib.wave_mxfp4_workspace_bytes.restype = sz
    lib.wave_mxfp4_gemm_static.argtypes = [p, p, p, p, p, i64, i64, i64, i32, i32, i32, i32, i32, i32, p]
    lib.wave_mxfp4_gemm_static.restype = i32
    lib.wave_mxfp4_static_scratch_bytes.argtypes = []
    lib.wave_mxfp4_static_scratch_bytes.restype = sz
    lib.wave_mxfp4_gemm_grouped.argtypes = [p, p, p, p, p, p, i32, i64, i64, i64, i32, i32, i32, i32, i32, p, sz, p]
    lib.wave_mxfp4_grouped_workspace_bytes.argtypes = [i64, i64, i64, i32]
    lib.wave_mxfp4_grouped_workspace_bytes.restype = sz
    lib.wave_mxfp4_gemm_grouped.restype = i32
    lib.wave_mxfp8_gemm.argtypes = [p, p, p, p, p, i64, i64, i64, i32, i32, i32, p, sz, i32, p]
    lib.wave_mxfp8_workspace_bytes.argtypes = [i64, i64, i64]
    lib.wave_mxfp8_workspace_bytes.restype = sz
    lib.wave_mxfp8_gemm.restype = i32
    lib.wave_mxfp8_b_preshuffle.argtypes = [p, p, i64, i64, p]
    lib.wave_mxfp8_b_preshuffle.restype = i32
    lib.wave_mxfp8_gemm_b_preshuffled.argtypes = [p, p, p, p, p, i64, i64, i64, i32, i32, i32, i32, i32, p, sz, p]
    lib.wave_mxfp8_gemm_b_preshuffled.restype = i32
    lib.wave_mxfp4_to_f32.argtypes = [p, p, i64, i64, p]
    lib.wave_mxfp4_to_f32.restype = i32
    lib.wave_mxfp4_e8m0_to_f32.argtypes = [p, p, i64, p]
    lib.wave_mxfp4_e8m0_to_f32.restype = i32
    lib.wave_mxfp4_dequant.argtypes = [p, p, p, i64, i64, i32, p]
    lib.wave_mxfp4_dequant.restype = i32
    lib.wave_mxfp4_e8m0_shuffle.argtypes = [p, p, i64, i64, p]
    lib.wave_mxfp4_e8m0_shuffle.restype = i32
    lib.wave_mxfp4_e8m0_shuffle_bytes.argtypes = [i64, i64]
    lib.wave_mxfp4_e8m0_shuffle_bytes.restype = sz
    lib.wave_mxfp4_scale_convert.argtypes = [p, i32, p, i32, i64, i64, p]
    lib.wave_mxfp4_scale_convert.restype = i32
    lib.wave_mxfp4_b_preshuffle.argtypes = [p, p, i64, i64, p]
    lib.wave_mxfp4_b_preshuffle.restype = i32
    lib.wave_mxfp4_quantize.argtypes = [p, i32, p, p, i64, i64, i32, p]
    lib.wave_mxfp4_quantize.restype = i32
    lib.wave_mxfp4_quantize_rows.argtypes = [p, i32, i64, p, i32, p, p, i64, i64, i32, p]
    lib.wave_mxfp4_quantize_rows.restype = i32
    lib.wave_mxfp4_moe_align_block_size.argtypes = [p, i32, i64, i32, i32, p, i64, p, i64, p, p, p]
    lib.wave_mxfp4_moe_align_block_size.restype = i32
    lib.wave_mxfp4_silu_and_mul.argtypes = [p, p, p, i64, i64, i64, i32, i64, i64, p]
    lib.wave_mxfp4_silu_and_mul.restype = i32
    lib.wave_mxfp4_silu_and_mul_quantize.argtypes = [p, p, i64, i64, i32, p, p, i64, i64, i32, p]
    lib.wave_mxfp4_silu_and_mul_quantize.restype = i32
    lib.wave_mxfp4_gemm_gated_quantize.argtypes = [p, p, p, p, p, p, p, i32, i64, i64, i64, i32, i32, i32, p, sz, p]
    lib.wave_mxfp4_gemm_gated_quantize.restype = i32
    lib.wave_mxfp4_interleave_gate_up.argtypes = [p, p, i64, i64, p]
    lib.wave_mxfp4_interleave_gate_up.restype = i32
    lib.wave_mxfp4_status_string.argtypes = [i32]
    lib.wave_mxfp4_status_string.restype = ctypes.c_char_p
    lib.wave_mxfp4_last_hip_error.argtypes = []
    lib.wave_mxfp4_last_hip_error.restype = ctypes.c_char_p
    lib.wave_mxfp4_abi_version.argtypes = []
    lib.wave_mxfp4_abi_version.restype = i32
    got = lib.wave_mxfp4_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH}: ABI version {got}, this package expects {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    """Turn a status code into the exception the reference would raise:
    argument problems are ValueError (wave_lang/kernel/wave/compile.py:1489-1500,
    templates/tagged_mxfp4_gemm.py:637-645), HIP failures RuntimeError
    (wave_lang/kernel/wave/runtime/runtime.cpp:96-109)."""
    if status == OK:
        return
    lib = load()
    text = lib.wave_mxfp4_status_string(status).decode()
    if status == ERR_HIP:
        raise RuntimeError(f"{what}: {text}: {lib.wave_mxfp4_last_hip_error().decode()}")
    raise ValueError(f"{what}: {text} (status {status})")
