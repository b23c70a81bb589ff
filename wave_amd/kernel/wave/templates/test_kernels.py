"""The two scaled-GEMM variants the reference keeps outside its tagged
templates, with the reference's names and return conventions.

* ``get_broadcasted_scale_gemm_mxfp4`` (wave_lang/kernel/wave/templates/
  test_kernels.py:75-135): ``a_scale`` is ``[M]``, one e8m0 byte per row held
  for every 32-group of the row.  Returns ``(kernel, hyperparams)`` as the
  reference does; the caller builds the options from the hyperparameters.
* ``get_batched_scaled_gemm_template`` (tests/kernel/wave_gemm_mxfp_test.py:
  205-299): ``a [B, M, K/2]`` with a shared ``b [N, K/2]``, output
  ``[B, M, N]`` f32.  Returns ``(options, kernel)`` as the reference's helper
  does."""

from __future__ import annotations

from ... import lang as tkl
from .... import _lib
from ..compile import KernelSpec, WaveCompileOptions
from ..constraints import ScaledMMAType


def get_broadcasted_scale_gemm_mxfp4(shape, mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4):
    spec = KernelSpec("broadcasted_scale_scaled_mma", tuple(shape), (32, 32, 256), (2, 2), tkl.f32,
                      a_scale_layout=_lib.SCALE_PER_ROW)
    hyperparams = {"BLOCK_M": 32, "BLOCK_N": 32, "BLOCK_K": 256, "M": shape[0], "N": shape[1], "K": shape[2]}
    return spec, hyperparams


def get_batched_scaled_gemm_template(shape, mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                     enable_scheduling=None):
    spec = KernelSpec("batched_gemm", tuple(shape), (256, 128, 256), (4, 2), tkl.f32)
    subs = {"BLOCK_B": 1, "BLOCK_M": 256, "BLOCK_N": 128, "BLOCK_K": 256, "N": shape[1], "K": shape[2]}
    options = WaveCompileOptions(subs=subs, canonicalize=True, schedule=enable_scheduling,
                                 dynamic_symbols=["B", "M"])
    return options, spec
