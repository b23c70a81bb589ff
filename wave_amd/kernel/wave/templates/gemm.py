"""``get_scaled_gemm_kernel`` with the reference's name, arguments and return
convention (wave_lang/kernel/wave/templates/gemm.py:134-205): the plain MXFP4
scaled GEMM, ``a [M, K/2]``, ``a_scale [M, K/32]``, ``b [N, K/2]``,
``b_scale [N, K/32]`` -> ``c [M, N]`` f32.  Returns ``(kernel, hyperparams)``;
the caller builds ``WaveCompileOptions(subs=hyperparams)`` and compiles, as
tests/kernel/wave/water_e2e_test.py:175-215 does.  The tile sizes only select
one of the prebuilt kernels (the reference's default 32x32x256 block has no
counterpart here and leaves the choice to the library)."""

from __future__ import annotations

from typing import Optional

from ... import lang as tkl
from ..compile import KernelSpec, select_variant
from ..constraints import ScaledMMAType


def get_scaled_gemm_kernel(shape: tuple, mfma_variant: ScaledMMAType = ScaledMMAType.F32_16x16x128_F8F6F4,
                           block_shape: Optional[tuple] = None, waves_per_block: Optional[tuple] = None):
    if len(shape) != 3:
        raise ValueError("shape is (M, N, K)")
    if not isinstance(mfma_variant, ScaledMMAType):
        raise ValueError("mfma_variant must be a ScaledMMAType")
    if not block_shape:
        block_shape = (32, 32, 256)
    if not waves_per_block:
        waves_per_block = (2, 2)
    if shape[2] % 32 != 0:
        raise ValueError(f"K = {shape[2]} must be a multiple of 32")
    spec = KernelSpec("scaled_gemm", tuple(shape), tuple(block_shape), tuple(waves_per_block), tkl.f32,
                      variant=select_variant(block_shape, waves_per_block))
    hyperparams = {"BLOCK_M": block_shape[0], "BLOCK_N": block_shape[1], "BLOCK_K": block_shape[2],
                   "M": shape[0], "N": shape[1], "K": shape[2]}
    return spec, hyperparams
