"""``wave_compile`` and ``WaveKernel`` for the MXFP4 scaled-GEMM templates.

In the reference ``wave_compile(options, kernel, schedule)`` traces the
template, runs the compiler and loads the generated code object
(wave_lang/kernel/wave/compile.py:1021-1090); the returned ``WaveKernel`` is
called with torch tensors and launches on the current stream
(compile.py:225-339).  Here the kernels are prebuilt HIP, so "compiling" only
selects one of them from the template's parameters."""

from __future__ import annotations

import dataclasses

from dataclasses import dataclass, field
from typing import Any

from .. import lang as tkl
from ... import _lib
from ... import mxfp4 as _ops


@dataclass
class WaveCompileOptions:
    """The subset of the reference's option block
    (wave_lang/kernel/wave/compile_options.py:18-160) the scaled-GEMM path
    reads; unknown keyword arguments are kept in ``extra``."""

    subs: dict = field(default_factory=dict)
    canonicalize: bool = True
    schedule: Any = None
    use_global_to_shared: bool = True
    minimize_shared_allocs: bool = False
    dynamic_symbols: list = field(default_factory=list)
    extra: dict = field(default_factory=dict)


@dataclass
class KernelSpec:
    """What a template getter hands to ``wave_compile``."""

    name: str
    shape: tuple
    block_shape: tuple
    wave_shape: tuple
    output_dtype: Any = tkl.f32
    a_scale_layout: int = _lib.SCALE_ROW_MAJOR
    b_scale_layout: int = _lib.SCALE_ROW_MAJOR
    b_layout: int = _lib.B_ROW_MAJOR
    num_splits: int = 1
    variant: int = _lib.VARIANT_AUTO


_TILE_VARIANTS = {
    ((256, 256), (2, 2)): _lib.VARIANT_T256x256_W2x2,
    ((256, 256), (4, 2)): _lib.VARIANT_T256x256_W4x2,
    ((128, 128), (2, 2)): _lib.VARIANT_T128x128_W2x2,
    ((128, 256), (2, 2)): _lib.VARIANT_T128x256_W2x2,
}


def select_variant(block_shape, wave_shape) -> int:
    """(BLOCK_M, BLOCK_N, BLOCK_K) x (WAVE_M, WAVE_N) -> prebuilt kernel.  Tile
    shapes that were not built fall back to the library's own choice."""
    key = ((int(block_shape[0]), int(block_shape[1])), (int(wave_shape[0]), int(wave_shape[1])))
    return _TILE_VARIANTS.get(key, _lib.VARIANT_AUTO)


class WaveKernel:
    """Callable with the reference's calling convention:
    ``kernel(x, x_scales, w_t, w_scales, out)`` -> None, ``out`` mutated in
    place on the current stream (wave_lang/kernel/wave/compile.py:225-339)."""

    def __init__(self, spec: KernelSpec, options: WaveCompileOptions, schedule=None):
        self.spec = spec
        self.options = options
        self.schedule = schedule

    def __call__(self, x, x_scales, w_t, w_scales, out):
        s = self.spec
        want = s.output_dtype.torch_dtype
        if out.dtype != want:
            raise ValueError(f"kernel was built for {want} output, got {out.dtype}")
        split = s.num_splits if s.num_splits > 1 else 0  # a plain template leaves the choice to the library
        if split > 1:
            # The library splits K in whole 256-element tiles; take the largest
            # split count not above the requested one that does.
            k = x.shape[-1] * 2
            while split > 1 and (k % split != 0 or (k // split) % 256 != 0):
                split -= 1
        _ops.mxfp4_gemm(x, x_scales, w_t, w_scales, out, a_scale_layout=s.a_scale_layout,
                        b_scale_layout=s.b_scale_layout, b_layout=s.b_layout, split_k=split,
                        variant=s.variant)
        return None

    invoke = __call__


def wave_compile(options: WaveCompileOptions, kernel: KernelSpec, schedule=None) -> WaveKernel:
    if not isinstance(kernel, KernelSpec):
        raise TypeError("wave_compile expects the kernel object returned by a template getter")
    _lib.load()  # fail here, not at first launch, if the HIP library is missing
    # The asymmetric schedule of the reference (A through LDS, preshuffled B straight into registers,
    # schedules/gemm_mxfp4_double_buffer.py:1781-2222) names a kernel of its own here: the B-direct variant, where
    # the template's shape allows it (256 x 256 tiles, whole 256-column tiles, an even number of at least 6 K
    # tiles); every other schedule is pipelining the hand-written kernels already fix.
    if (getattr(schedule, "name", None) == "mxfp4_asymmetric" and kernel.b_layout == _lib.B_PRESHUFFLE
            and kernel.num_splits <= 1 and tuple(kernel.block_shape[:2]) == (256, 256)
            and kernel.shape[1] % 256 == 0 and kernel.shape[2] % 512 == 0 and kernel.shape[2] >= 1536):
        kernel = dataclasses.replace(kernel, variant=_lib.VARIANT_T256x256_W1x4_BDIRECT)
    return WaveKernel(kernel, options, schedule)
