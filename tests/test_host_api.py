"""Host-side mirror of the reference interface (no GPU): template getters,
their argument checks and error messages, variant selection, CPU layout
helpers against the oracle."""

import numpy as np
import pytest
import torch

import wave_amd.kernel.lang as tkl
from oracle import mxfp4_oracle as orc
from wave_amd import _lib
from wave_amd.kernel.wave.compile import WaveCompileOptions, wave_compile
from wave_amd.kernel.wave.constraints import ScaledMMAType
from wave_amd.kernel.wave.schedules import (
    get_mxfp4_asymmetric_schedule,
    get_mxfp4_dbuf_pingpong_schedule,
    get_mxfp4_dbuf_schedule,
)
from wave_amd.kernel.wave.templates import (
    get_tagged_mxfp4_gemm,
    get_tagged_mxfp4_gemm_preshuffle_b,
    get_tagged_mxfp4_gemm_preshuffle_b_wide_store,
    get_tagged_mxfp4_gemm_preshuffle_scales,
    get_tagged_mxfp4_gemm_preshuffle_scales_and_B,
    get_tagged_splitk_mxfp4_gemm,
)
from wave_amd.kernel.wave.utils.mxfp_utils import (
    SCALE_GROUP_SIZE,
    b_preshuffle,
    e8m0_shuffle,
    generate_gemm_afp4wfp4_inputs,
)


def test_plain_template_selects_prebuilt_kernels():
    for block, waves, want in [((256, 256, 256), (2, 2), _lib.VARIANT_T256x256_W2x2),
                               ((256, 256, 256), (4, 2), _lib.VARIANT_T256x256_W4x2),
                               ((128, 128, 256), (2, 2), _lib.VARIANT_T128x128_W2x2),
                               ((256, 192, 256), (2, 2), _lib.VARIANT_AUTO)]:
        spec, options = get_tagged_mxfp4_gemm((1024, 1024, 8192), block, wave_shape=waves,
                                              mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4)
        assert spec.variant == want
        assert isinstance(options, WaveCompileOptions)
        assert options.subs["BLOCK_M"] == block[0]
        k = wave_compile(options, spec, get_mxfp4_dbuf_schedule(use_stagger=False))
        assert callable(k)


def test_variant_layouts():
    s, _ = get_tagged_mxfp4_gemm_preshuffle_scales((1024, 1024, 8192))
    assert (s.a_scale_layout, s.b_scale_layout, s.b_layout) == (1, 1, 0)
    s, _ = get_tagged_mxfp4_gemm_preshuffle_scales_and_B((1024, 1024, 8192), output_dtype=tkl.bf16)
    assert (s.a_scale_layout, s.b_scale_layout, s.b_layout) == (1, 1, 1)
    assert s.output_dtype is tkl.bf16
    s, _ = get_tagged_mxfp4_gemm_preshuffle_b((1024, 1024, 8192), a_scale_preshuffle=False)
    assert (s.a_scale_layout, s.b_scale_layout, s.b_layout) == (0, 1, 1)
    s, _ = get_tagged_mxfp4_gemm_preshuffle_b_wide_store((1024, 3072, 8192))
    assert s.output_dtype is tkl.bf16 and s.b_layout == 1
    get_mxfp4_dbuf_pingpong_schedule(use_stagger=True, shape=(1, 2, 3))
    get_mxfp4_asymmetric_schedule(eliminate_epilogue=True)


def test_unsupported_output_dtype_asserts():
    with pytest.raises(AssertionError, match="Unsupported output dtype"):
        get_tagged_mxfp4_gemm(output_dtype=tkl.i8)


def test_splitk_rules_and_messages():
    # same rules and texts as the reference's template
    with pytest.raises(ValueError, match=r"K per split \(128\) is less than BLOCK_K \(256\)"):
        get_tagged_splitk_mxfp4_gemm((256, 256, 512), num_splits=4, block_shape=(128, 128, 256))
    with pytest.raises(ValueError, match=r"k_per_split \(384\) must be a multiple of BLOCK_K \(256\)"):
        get_tagged_splitk_mxfp4_gemm((256, 256, 768), num_splits=2, block_shape=(128, 128, 256))
    s, _ = get_tagged_splitk_mxfp4_gemm((256, 256, 1024), num_splits=4, block_shape=(128, 128, 128),
                                        output_type=tkl.bf16)
    assert s.num_splits == 4 and s.output_dtype is tkl.bf16


def test_kernel_rejects_wrong_output_dtype():
    spec, options = get_tagged_mxfp4_gemm((64, 64, 256))
    k = wave_compile(options, spec)
    z = torch.zeros(64, 128, dtype=torch.uint8)
    with pytest.raises(ValueError, match="built for torch.float32"):
        k(z, z, z, z, torch.zeros(64, 64, dtype=torch.bfloat16))
    with pytest.raises(TypeError):
        wave_compile(options, object())


def test_operators_refuse_cpu_tensors():
    import wave_amd

    z = torch.zeros(64, 128, dtype=torch.uint8)
    s = torch.zeros(64, 8, dtype=torch.uint8)
    with pytest.raises(ValueError, match="no CPU path"):
        wave_amd.mxfp4_gemm(z, s, z, s, torch.zeros(64, 64))
    with pytest.raises(ValueError, match="no CPU path"):
        wave_amd.mxfp4_to_f32(z)


def test_generator_shapes_and_ranges():
    x, w, xs, ws = generate_gemm_afp4wfp4_inputs((64, 96, 256), device=torch.device("cpu"))
    assert x.shape == (64, 128) and w.shape == (128, 96) and not w.is_contiguous()
    assert xs.shape == (64, 8) and ws.shape == (96, 8) and xs.is_contiguous()
    assert xs.min() >= 124 and xs.max() <= 127 and SCALE_GROUP_SIZE == 32
    x2, *_ = generate_gemm_afp4wfp4_inputs((64, 96, 256), device=torch.device("cpu"))
    assert torch.equal(x, x2)


def test_cpu_layout_helpers_match_oracle():
    rng = np.random.default_rng(0)
    b = rng.integers(0, 256, size=(48, 96), dtype=np.uint8)
    assert np.array_equal(b_preshuffle(torch.from_numpy(b)).numpy(), orc.b_preshuffle(b))
    s = rng.integers(0, 256, size=(96, 16), dtype=np.uint8)
    got = e8m0_shuffle(torch.from_numpy(s)).numpy()
    assert np.array_equal(got, orc.e8m0_shuffle_padded(s)[:96])
    s = rng.integers(0, 256, size=(256, 32), dtype=np.uint8)
    assert np.array_equal(e8m0_shuffle(torch.from_numpy(s)).numpy(), orc.e8m0_shuffle(s))


def test_superseded_scratch_buffers_stay_alive():
    """A buffer that was handed out may sit in a captured HIP graph: growing the cache must not free it."""
    import weakref

    from wave_amd import mxfp4 as host

    key = ("test-device", 12345)
    made = []

    def alloc(n):
        t = torch.empty(n, dtype=torch.uint8)
        made.append(weakref.ref(t))
        return t

    try:
        small = host._grow_scratch(key, 100, alloc)
        assert host._grow_scratch(key, 50, alloc) is small          # large enough: reused
        ptr = small.data_ptr()
        big = host._grow_scratch(key, 1000, alloc)
        assert big is not small and big.numel() == 1024  # grown geometrically: the next power of two
        del small
        assert made[0]() is not None and made[0]().data_ptr() == ptr  # still referenced by the module
        assert host._grow_scratch(key, 1000, alloc) is big
        # a run of slowly growing requests retires less than the live buffer holds
        before = len(host._retired)
        for n in range(1025, 9000, 7):
            last = host._grow_scratch(key, n, alloc)
        retired = sum(t.numel() for t in host._retired[before:])
        assert retired < last.numel() and last.numel() == 16384
    finally:
        host._scratch.pop(key, None)


def test_asymmetric_schedule_selects_the_b_direct_kernel():
    """wave_compile(options, preshuffle-B template, get_mxfp4_asymmetric_schedule()) names the kernel that keeps A in
    LDS and reads preshuffled B straight into registers, where the shape allows; other schedules, shapes and
    templates keep their (block_shape, wave_shape) choice."""
    spec, options = get_tagged_mxfp4_gemm_preshuffle_b((1024, 1024, 8192), (256, 256, 256), wave_shape=(2, 2))
    assert wave_compile(options, spec, get_mxfp4_asymmetric_schedule()).spec.variant == _lib.VARIANT_T256x256_W1x4_BDIRECT
    assert wave_compile(options, spec, get_mxfp4_dbuf_schedule()).spec.variant == _lib.VARIANT_T256x256_W2x2
    assert spec.variant == _lib.VARIANT_T256x256_W2x2                       # the template object is left as it was
    for shape, block in [((1024, 1024, 1024), (256, 256, 256)),             # K too short
                         ((1024, 3072, 8192), (256, 192, 256)),             # another tile
                         ((512, 768, 2304), (256, 256, 256))]:              # an odd number of K tiles
        spec, options = get_tagged_mxfp4_gemm_preshuffle_b(shape, block, wave_shape=(2, 2))
        k = wave_compile(options, spec, get_mxfp4_asymmetric_schedule())
        assert k.spec.variant != _lib.VARIANT_T256x256_W1x4_BDIRECT
    spec, options = get_tagged_mxfp4_gemm((1024, 1024, 8192), (256, 256, 256), wave_shape=(2, 2))
    assert wave_compile(options, spec, get_mxfp4_asymmetric_schedule()).spec.variant == _lib.VARIANT_T256x256_W2x2
