from .gemm import get_scaled_gemm_kernel
from .tagged_mxfp4_gemm import (
    get_tagged_mxfp4_gemm,
    get_tagged_mxfp4_gemm_preshuffle_b,
    get_tagged_mxfp4_gemm_preshuffle_b_wide_store,
    get_tagged_mxfp4_gemm_preshuffle_scales,
    get_tagged_mxfp4_gemm_preshuffle_scales_and_B,
    get_tagged_splitk_mxfp4_gemm,
    get_tagged_splitk_mxfp4_gemm_preshuffle_b,
    get_tagged_splitk_mxfp4_gemm_preshuffle_scales,
)
from .test_kernels import get_batched_scaled_gemm_template, get_broadcasted_scale_gemm_mxfp4

__all__ = [
    "get_batched_scaled_gemm_template",
    "get_broadcasted_scale_gemm_mxfp4",
    "get_scaled_gemm_kernel",
    "get_tagged_mxfp4_gemm",
    "get_tagged_mxfp4_gemm_preshuffle_b",
    "get_tagged_mxfp4_gemm_preshuffle_b_wide_store",
    "get_tagged_mxfp4_gemm_preshuffle_scales",
    "get_tagged_mxfp4_gemm_preshuffle_scales_and_B",
    "get_tagged_splitk_mxfp4_gemm",
    "get_tagged_splitk_mxfp4_gemm_preshuffle_b",
    "get_tagged_splitk_mxfp4_gemm_preshuffle_scales",
]
