"""Template getters of the MXFP4 scaled GEMM, same names and arguments as
wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py.  Each returns
``(kernel, options)`` for ``wave_compile``; the kernel it stands for takes
``(a [M,K/2] u8, a_scale, b [N,K/2] u8, b_scale, c [M,N])``.

What the variants mean here:
* plain (:38-145)                 - A, B, scales row-major.
* preshuffle_scales (:334-365)    - both scale tensors in ``e8m0_shuffle`` order.
* preshuffle_scales_and_B (:368-403) - plus B in ``b_preshuffle`` order.
* preshuffle_b (:950-991)         - B preshuffled, B scales shuffled, A scales
                                    shuffled iff ``a_scale_preshuffle``.
* preshuffle_b_wide_store (:994-1035) - same inputs; all kernels here already
                                    store 8/16 bytes per lane.
* splitk (:819-947)               - K split over workgroups.  The reference adds
                                    partial sums into a zero-initialised C with
                                    atomics; here partials are kept in f32 and C
                                    is overwritten with their sum, so a zeroed C
                                    gives the same result (and bf16 output is
                                    rounded once, not once per split).
``mfma_variant``, address spaces, workgroup reordering and ``group_size_n``
are accepted for compatibility; the kernels use the 32x32x64 scaled MFMA and
their own XCD-aware tile order."""

from __future__ import annotations

import math

from ... import lang as tkl
from ...lang import SHARED_ADDRESS_SPACE
from .... import _lib
from ..compile import KernelSpec, WaveCompileOptions, select_variant
from ..constraints import ScaledMMAType


def _options(shape, block_shape):
    subs = {"M": shape[0], "N": shape[1], "K": shape[2], "BLOCK_M": block_shape[0],
            "BLOCK_N": block_shape[1], "BLOCK_K": block_shape[2]}
    return WaveCompileOptions(subs=subs, canonicalize=True, schedule="manual", use_global_to_shared=True,
                              minimize_shared_allocs=False)


def _check_out(output_dtype):
    assert output_dtype in [tkl.f32, tkl.bf16], f"Unsupported output dtype: {output_dtype}"


def get_tagged_mxfp4_gemm(shape=(1024, 1024, 8192), block_shape=(256, 256, 256), wave_shape=(2, 2),
                          mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                          a_address_space=SHARED_ADDRESS_SPACE, b_address_space=SHARED_ADDRESS_SPACE,
                          reorder_workgroups=True, group_size_n=32, output_dtype=tkl.f32):
    _check_out(output_dtype)
    spec = KernelSpec("mxfp4_gemm", tuple(shape), tuple(block_shape), tuple(wave_shape), output_dtype,
                      variant=select_variant(block_shape, wave_shape))
    return spec, _options(shape, block_shape)


def _check_shuffled_shape(shape, what):
    # the reference's templates assume this for the shuffled layouts
    # (tagged_mxfp4_gemm.py:190-201,445-451)
    m, n, k = shape
    if k % 256 != 0:
        raise ValueError(f"{what}: K = {k} must be a multiple of 256 for preshuffled scales")
    if n % 32 != 0:
        raise ValueError(f"{what}: N = {n} must be a multiple of 32 for preshuffled scales")


def get_tagged_mxfp4_gemm_preshuffle_scales(shape=(1024, 1024, 8192), block_shape=(256, 256, 256),
                                            wave_shape=(2, 2),
                                            mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                            a_address_space=SHARED_ADDRESS_SPACE):
    _check_shuffled_shape(shape, "preshuffle_scales")
    spec = KernelSpec("mxfp4_gemm_preshuffle_scales", tuple(shape), tuple(block_shape), tuple(wave_shape),
                      tkl.f32, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                      variant=select_variant(block_shape, wave_shape))
    return spec, _options(shape, block_shape)


def get_tagged_mxfp4_gemm_preshuffle_scales_and_B(shape=(1024, 1024, 8192), block_shape=(256, 256, 256),
                                                  wave_shape=(2, 2),
                                                  mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                                  a_address_space=SHARED_ADDRESS_SPACE,
                                                  b_address_space=None, output_dtype=tkl.f32):
    _check_out(output_dtype)
    _check_shuffled_shape(shape, "preshuffle_scales_and_B")
    spec = KernelSpec("mxfp4_gemm_preshuffle_scales_and_B", tuple(shape), tuple(block_shape),
                      tuple(wave_shape), output_dtype, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                      b_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_layout=_lib.B_PRESHUFFLE,
                      variant=select_variant(block_shape, wave_shape))
    return spec, _options(shape, block_shape)


def get_tagged_mxfp4_gemm_preshuffle_b(shape=(1024, 1024, 8192), block_shape=(256, 256, 256),
                                       wave_shape=(2, 2),
                                       mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                       a_address_space=SHARED_ADDRESS_SPACE, a_scale_preshuffle=True,
                                       reorder_workgroups=True, group_size_n=32, output_dtype=tkl.f32):
    _check_out(output_dtype)
    _check_shuffled_shape(shape, "preshuffle_b")
    spec = KernelSpec("mxfp4_gemm_preshuffle_b", tuple(shape), tuple(block_shape), tuple(wave_shape),
                      output_dtype,
                      a_scale_layout=_lib.SCALE_E8M0_SHUFFLE if a_scale_preshuffle else _lib.SCALE_ROW_MAJOR,
                      b_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_layout=_lib.B_PRESHUFFLE,
                      variant=select_variant(block_shape, wave_shape))
    return spec, _options(shape, block_shape)


def get_tagged_mxfp4_gemm_preshuffle_b_wide_store(shape=(1024, 1024, 8192), block_shape=(256, 256, 256),
                                                  wave_shape=(2, 2),
                                                  mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                                  a_address_space=SHARED_ADDRESS_SPACE,
                                                  a_scale_preshuffle=True, reorder_workgroups=True,
                                                  group_size_n=32, output_dtype=tkl.bf16):
    spec, options = get_tagged_mxfp4_gemm_preshuffle_b(shape, block_shape, wave_shape, mfma_variant,
                                                       a_address_space, a_scale_preshuffle,
                                                       reorder_workgroups, group_size_n, output_dtype)
    spec.name = "mxfp4_gemm_preshuffle_b_wide_store"
    return spec, options


def _splitk(shape, num_splits, block_shape, wave_shape, output_type, *, preshuffle_scales=False,
            preshuffle_B=False):
    _check_out(output_type)
    m, n, k = shape
    # same checks and messages as the reference (tagged_mxfp4_gemm.py:636-645)
    k_per_split = math.ceil(k / num_splits)
    if k_per_split < block_shape[2]:
        raise ValueError(
            f"K per split ({k_per_split}) is less than BLOCK_K ({block_shape[2]}). "
            f"Reduce num_splits or BLOCK_K so that each split has at least BLOCK_K elements.")
    if k_per_split % block_shape[2] != 0:
        raise ValueError(f"k_per_split ({k_per_split}) must be a multiple of BLOCK_K ({block_shape[2]}).")
    shuffled = preshuffle_scales or preshuffle_B
    if shuffled:
        _check_shuffled_shape(shape, "splitk")
    spec = KernelSpec("splitk_mxfp4_gemm", tuple(shape), tuple(block_shape), tuple(wave_shape), output_type,
                      a_scale_layout=_lib.SCALE_E8M0_SHUFFLE if shuffled else _lib.SCALE_ROW_MAJOR,
                      b_scale_layout=_lib.SCALE_E8M0_SHUFFLE if shuffled else _lib.SCALE_ROW_MAJOR,
                      b_layout=_lib.B_PRESHUFFLE if preshuffle_B else _lib.B_ROW_MAJOR,
                      num_splits=int(num_splits), variant=select_variant(block_shape, wave_shape))
    if spec.variant == _lib.VARIANT_AUTO:
        spec.variant = _lib.VARIANT_T128x128_W2x2
    return spec, _options(shape, block_shape)


def get_tagged_splitk_mxfp4_gemm(shape=(1024, 1024, 8192), num_splits=2, block_shape=(128, 128, 256),
                                 wave_shape=(2, 2), mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                 a_address_space=SHARED_ADDRESS_SPACE, output_type=tkl.f32):
    return _splitk(shape, num_splits, block_shape, wave_shape, output_type)


def get_tagged_splitk_mxfp4_gemm_preshuffle_scales(shape=(1024, 1024, 8192), num_splits=2,
                                                   block_shape=(128, 128, 256), wave_shape=(2, 2),
                                                   mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                                   a_address_space=SHARED_ADDRESS_SPACE,
                                                   output_type=tkl.f32):
    return _splitk(shape, num_splits, block_shape, wave_shape, output_type, preshuffle_scales=True)


def get_tagged_splitk_mxfp4_gemm_preshuffle_b(shape=(1024, 1024, 8192), num_splits=2,
                                              block_shape=(128, 128, 256), wave_shape=(2, 2),
                                              mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                              a_address_space=SHARED_ADDRESS_SPACE, output_type=tkl.f32):
    return _splitk(shape, num_splits, block_shape, wave_shape, output_type, preshuffle_B=True)
