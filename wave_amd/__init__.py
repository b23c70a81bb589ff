"""wave_amd: MI355X-native MXFP4 block-scaled GEMM behind the calling
convention of the reference's scaled-GEMM kernels
(``gemm(x, x_scales, w_t, w_scales, out)``)."""

from . import _lib
from .mxfp4 import (
    b_preshuffle,
    dequant,
    e8m0_shuffle,
    e8m0_to_f32,
    interleave_gate_up,
    mxfp4_gemm,
    mxfp4_gemm_gated_quantize,
    mxfp4_gemm_grouped,
    moe_align_block_size,
    mxfp4_to_f32,
    mxfp8_b_preshuffle,
    mxfp8_gemm,
    quantize_mxfp4,
    quantize_mxfp4_rows,
    silu_and_mul,
    silu_and_mul_quantize,
    scale_convert,
    workspace_bytes,
)

__all__ = [
    "b_preshuffle",
    "dequant",
    "e8m0_shuffle",
    "e8m0_to_f32",
    "interleave_gate_up",
    "mxfp4_gemm",
    "mxfp4_gemm_gated_quantize",
    "mxfp4_gemm_grouped",
    "moe_align_block_size",
    "mxfp4_to_f32",
    "mxfp8_b_preshuffle",
    "mxfp8_gemm",
    "quantize_mxfp4",
    "quantize_mxfp4_rows",
    "silu_and_mul",
    "silu_and_mul_quantize",
    "scale_convert",
    "workspace_bytes",
]
