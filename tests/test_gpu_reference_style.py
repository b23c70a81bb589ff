"""The reference's own end-to-end tests of this path, re-expressed against the
mirrored interface (wave_lang -> wave_amd): same template getters, schedules,
``wave_compile``, input generator, call shape and tolerances
(tests/kernel/wave_gemm_mxfp_test.py:637-775,778-1085,
tests/kernel/wave_gemm_test.py:3641-3690).  The torch oracle is this
repository's port of the reference's ``torchScaledGemmMXFP4``."""

import pytest
import torch

import wave_amd.kernel.lang as tkl
from oracle.torch_oracle import torch_scaled_gemm_mxfp4
from wave_amd.kernel.lang import TORCH_DTYPE_TO_WAVE
from wave_amd.kernel.wave.compile import WaveCompileOptions, wave_compile
from wave_amd.kernel.wave.constraints import ScaledMMAType
from wave_amd.kernel.wave.schedules import (
    get_mxfp4_asymmetric_schedule,
    get_mxfp4_dbuf_pingpong_schedule,
    get_mxfp4_dbuf_pingpong_schedule_Bshuffled,
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
    b_preshuffle,
    e8m0_shuffle,
    generate_gemm_afp4wfp4_inputs,
)

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def torchScaledGemmMXFP4(x, w, x_scales, w_scales):
    """Reference signature: ``w`` is the transposed view [K/2, N]."""
    return torch_scaled_gemm_mxfp4(x.cpu(), w.T.contiguous().cpu(), x_scales.cpu(), w_scales.cpu())


@pytest.mark.parametrize("shape", [(1024, 1024, 8192)])
@pytest.mark.parametrize("block_shape", [(256, 256, 256)])
@pytest.mark.parametrize("wave_shape,use_stagger", [((2, 2), False), ((4, 2), True)])
def testScaledGemmMXFP4ManualDoubleBuf(shape, block_shape, wave_shape, use_stagger):
    gemm, options = get_tagged_mxfp4_gemm(shape, block_shape, wave_shape=wave_shape,
                                          mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4)
    gemm = wave_compile(options, gemm, get_mxfp4_dbuf_schedule(use_stagger=use_stagger))
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.float32, device=DEV)
    w_t = w.T.contiguous()
    gemm(x, x_scales, w_t, w_scales, out)
    torch_out = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    torch.testing.assert_close(torch_out, out.cpu(), check_dtype=False)


@pytest.mark.parametrize("shape", [(1024, 1024, 8192), (1024, 3072, 8192)])
def testScaledGemmMXFP4Bf16Output(shape):
    gemm, options = get_tagged_mxfp4_gemm(shape, (256, 256, 256), wave_shape=(2, 2), output_dtype=tkl.bf16)
    gemm = wave_compile(options, gemm, get_mxfp4_dbuf_schedule(use_stagger=False))
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.bfloat16, device=DEV)
    gemm(x, x_scales, w.T.contiguous(), w_scales, out)
    torch_out = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    torch.testing.assert_close(torch_out, out.cpu(), check_dtype=False)


@pytest.mark.parametrize("shape", [(1024, 1024, 8192), (256, 1024, 2048)])
def testScaledGemmMXFP4PreshuffleScales(shape):
    gemm, options = get_tagged_mxfp4_gemm_preshuffle_scales(shape, (256, 256, 256), wave_shape=(4, 2))
    gemm = wave_compile(options, gemm, get_mxfp4_dbuf_pingpong_schedule(use_stagger=True, shape=shape))
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.float32, device=DEV)
    gemm(x, e8m0_shuffle(x_scales), w.T.contiguous(), e8m0_shuffle(w_scales), out)
    torch_out = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    torch.testing.assert_close(torch_out, out.cpu(), check_dtype=False)


@pytest.mark.parametrize("shape", [(1024, 1024, 8192)])
@pytest.mark.parametrize("output_dtype", [tkl.f32, tkl.bf16])
def testScaledGemmMXFP4PreshuffleScalesAndB(shape, output_dtype):
    gemm, options = get_tagged_mxfp4_gemm_preshuffle_scales_and_B(shape, (256, 256, 256), wave_shape=(4, 2),
                                                                  output_dtype=output_dtype)
    gemm = wave_compile(options, gemm, get_mxfp4_dbuf_pingpong_schedule_Bshuffled(use_stagger=True, shape=shape))
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=output_dtype.torch_dtype, device=DEV)
    gemm(x, e8m0_shuffle(x_scales), b_preshuffle(w.T.contiguous()), e8m0_shuffle(w_scales), out)
    torch_out = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    torch.testing.assert_close(torch_out, out.cpu(), check_dtype=False)


@pytest.mark.parametrize("shape,block_shape", [((1024, 1024, 8192), (256, 256, 256)),
                                               ((512, 768, 4096), (128, 256, 256)),
                                               ((1024, 3072, 8192), (256, 192, 256))])
@pytest.mark.parametrize("a_scale_preshuffle", [True, False])
def testScaledGemmMXFP4PreshuffleB(shape, block_shape, a_scale_preshuffle):
    gemm, options = get_tagged_mxfp4_gemm_preshuffle_b(shape, block_shape, wave_shape=(2, 2),
                                                       a_scale_preshuffle=a_scale_preshuffle)
    gemm = wave_compile(options, gemm, get_mxfp4_asymmetric_schedule())
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.float32, device=DEV)
    xs_in = e8m0_shuffle(x_scales) if a_scale_preshuffle else x_scales
    gemm(x, xs_in, b_preshuffle(w.T.contiguous()), e8m0_shuffle(w_scales), out)
    torch_out = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    torch.testing.assert_close(torch_out, out.cpu(), check_dtype=False)


def testScaledGemmMXFP4PreshuffleBWideStore():
    shape = (1024, 3072, 8192)
    gemm, options = get_tagged_mxfp4_gemm_preshuffle_b_wide_store(shape, (256, 192, 256), wave_shape=(2, 2))
    gemm = wave_compile(options, gemm, get_mxfp4_asymmetric_schedule())
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.bfloat16, device=DEV)
    gemm(x, e8m0_shuffle(x_scales), b_preshuffle(w.T.contiguous()), e8m0_shuffle(w_scales), out)
    torch_out = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    torch.testing.assert_close(torch_out, out.cpu(), check_dtype=False)


@pytest.mark.parametrize("shape, num_splits", [((256, 256, 256), 2), ((256, 256, 512), 4),
                                               ((256, 256, 1024), 4), ((512, 512, 1024), 4)])
@pytest.mark.parametrize("output_type", [torch.float32, torch.bfloat16])
def testSplitKMxfp4Gemm(shape, num_splits, output_type):
    splitk_gemm, options = get_tagged_splitk_mxfp4_gemm(shape, num_splits=num_splits,
                                                        block_shape=(128, 128, 128),
                                                        mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4,
                                                        output_type=TORCH_DTYPE_TO_WAVE[output_type])
    splitk_gemm = wave_compile(options, splitk_gemm, get_mxfp4_dbuf_schedule(use_stagger=True, k_partitions=1))
    m, n, k = shape
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=torch.device("cpu"))
    torch_ref = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    c_gpu = torch.zeros(m, n, dtype=output_type, device=DEV)
    splitk_gemm(x.cuda(), x_scales.cuda(), w.T.contiguous().cuda(), w_scales.cuda(), c_gpu)
    if output_type == torch.float32:
        torch.testing.assert_close(c_gpu.cpu(), torch_ref, rtol=1e-3, atol=1e-2)
    else:
        torch.testing.assert_close(c_gpu.cpu().to(torch.float32), torch_ref, rtol=1e-1, atol=4.0)


def testScaledGemmMXFP4BatchedStyleM1():
    """The reference runs M = 1, K = 1664 through its generic kernel
    (tests/kernel/wave_gemm_mxfp_test.py:296); K is not a multiple of 256."""
    shape = (1, 1024, 1664)
    gemm, options = get_tagged_mxfp4_gemm(shape, (256, 256, 256), wave_shape=(2, 2))
    gemm = wave_compile(options, gemm)
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(1, 1024, dtype=torch.float32, device=DEV)
    gemm(x, x_scales, w.T.contiguous(), w_scales, out)
    torch.testing.assert_close(torchScaledGemmMXFP4(x, w, x_scales, w_scales), out.cpu(), check_dtype=False)


@pytest.mark.parametrize("shape", [(512, 512, 512)])
def testBroadcastedScaleGemmMXFP4(shape):
    """tests/kernel/wave_gemm_mxfp_test.py:594-634."""
    from wave_amd.kernel.wave.compile import WaveCompileOptions
    from wave_amd.kernel.wave.templates import get_broadcasted_scale_gemm_mxfp4

    broadcasted_scale_scaled_mma, hyperparams = get_broadcasted_scale_gemm_mxfp4(
        shape, ScaledMMAType.F32_16x16x128_F8F6F4)
    options = WaveCompileOptions(subs=hyperparams, canonicalize=True, schedule=None)
    broadcasted_scale_scaled_mma = wave_compile(options, broadcasted_scale_scaled_mma)
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.float32, device=DEV)
    compacted_x_scales = x_scales[:, 0].contiguous()
    w_t = w.T.contiguous()
    broadcasted_scale_scaled_mma(x, compacted_x_scales, w_t, w_scales, out)
    broadcasted_compacted_x_scales = compacted_x_scales.view(-1, 1).repeat(1, x_scales.shape[-1]).contiguous()
    torch_out = torchScaledGemmMXFP4(x, w, broadcasted_compacted_x_scales, w_scales)
    torch.testing.assert_close(torch_out, out.cpu(), check_dtype=False)


def test_scaled_gemm_kernel_template():
    """tests/kernel/wave/water_e2e_test.py:172-230: the plain template of templates/gemm.py, compiled from its
    hyperparameters and checked against the torch dequant + matmul."""
    from wave_amd.kernel.wave.templates.gemm import get_scaled_gemm_kernel

    shape = (1024, 1024, 1024)
    scaled_gemm, hyperparams = get_scaled_gemm_kernel(shape=shape, mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4)
    options = WaveCompileOptions(subs=hyperparams, canonicalize=True)
    compiled = wave_compile(options, scaled_gemm)
    x, w, x_scales, w_scales = generate_gemm_afp4wfp4_inputs(shape, device=DEV)
    out = torch.zeros(shape[0], shape[1], dtype=torch.float32, device=DEV)
    compiled(x, x_scales, w.T.contiguous(), w_scales, out)
    expected = torchScaledGemmMXFP4(x, w, x_scales, w_scales)
    torch.testing.assert_close(out.cpu(), expected, rtol=1e-3, atol=1e-3, check_dtype=False)


@pytest.mark.parametrize("batch", [4, 8])
@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (1, 16384, 1664)])
def testScaledBatchedGemmMXFP4(batch, shape):
    """tests/kernel/wave_gemm_mxfp_test.py:302-339 at its two small shapes, every element against the torch
    oracle (the (8192, 8192, 8192) shape: testScaledBatchedGemmMXFP4Large below; (16384, 16384, 16384) x batch 8
    would need an 8.6 GB f32 C per batch and is not run)."""
    from wave_amd.kernel.wave.templates import get_batched_scaled_gemm_template

    options, batched_gemm = get_batched_scaled_gemm_template(shape, ScaledMMAType.F32_16x16x128_F8F6F4, None)
    batched_gemm = wave_compile(options, batched_gemm)
    linearized_shape = (batch * shape[0], shape[1], shape[2])
    flat_x, w, flat_x_scales, w_scales = generate_gemm_afp4wfp4_inputs(linearized_shape, device=DEV)
    w_t = w.T.contiguous()
    x = flat_x.view(batch, shape[0], shape[2] // 2)
    x_scales = flat_x_scales.view(batch, shape[0], shape[2] // 32)
    w_t = w_t.view(shape[1], shape[2] // 2)
    w_scales = w_scales.view(shape[1], shape[2] // 32)
    out = torch.zeros(batch, shape[0], shape[1], dtype=torch.float32, device=DEV)
    batched_gemm(x, x_scales, w_t, w_scales, out)
    torch_flat_out = torchScaledGemmMXFP4(flat_x, w, flat_x_scales, w_scales)
    torch_out = torch_flat_out.view(batch, shape[0], shape[1])
    torch.testing.assert_close(torch_out, out.cpu())


def testScaledBatchedGemmMXFP4Large():
    """tests/kernel/wave_gemm_mxfp_test.py:302-339 at its (8192, 8192, 8192) shape, batch 4: 32768 rows of A
    against one B, f32 out.  The reference compares every element with torch on the GPU; here rows of every
    256-row M tile (8 per tile, all residues mod 32: 1024 rows) meet the exact C oracle under the reference's
    tolerance (torch.testing.assert_close defaults for f32: rtol 1.3e-6, atol 1e-5), and every batch must equal,
    bit for bit, the plain 2-D call on its own slice (the batch is folded into the rows)."""
    import numpy as np

    from oracle import c_oracle
    from wave_amd.kernel.wave.templates import get_batched_scaled_gemm_template

    batch, shape = 4, (8192, 8192, 8192)
    options, batched_gemm = get_batched_scaled_gemm_template(shape, ScaledMMAType.F32_16x16x128_F8F6F4, None)
    batched_gemm = wave_compile(options, batched_gemm)
    linearized_shape = (batch * shape[0], shape[1], shape[2])
    flat_x, w, flat_x_scales, w_scales = generate_gemm_afp4wfp4_inputs(linearized_shape, device=DEV)
    w_t = w.T.contiguous()
    x = flat_x.view(batch, shape[0], shape[2] // 2)
    x_scales = flat_x_scales.view(batch, shape[0], shape[2] // 32)
    out = torch.zeros(batch, shape[0], shape[1], dtype=torch.float32, device=DEV)
    batched_gemm(x, x_scales, w_t, w_scales, out)
    m = linearized_shape[0]
    rows = np.array(sorted({t * 256 + 32 * b + (4 * b + t) % 32 for t in range(m // 256) for b in range(8)}
                           | {0, 255, 256, m - 1}))
    assert set(rows % 32) == set(range(32))
    ref = c_oracle.scaled_gemm_exact(flat_x.cpu().numpy(), w_t.cpu().numpy(), flat_x_scales.cpu().numpy(),
                                     w_scales.cpu().numpy(), rows=rows)
    got = out.view(m, shape[1])[torch.from_numpy(rows).to(DEV)].cpu()
    torch.testing.assert_close(got, torch.from_numpy(ref).float())
    gemm2d, opt2d = get_tagged_mxfp4_gemm(shape, (256, 256, 256), wave_shape=(4, 2),
                                          mfma_variant=ScaledMMAType.F32_16x16x128_F8F6F4)
    gemm2d = wave_compile(opt2d, gemm2d, get_mxfp4_dbuf_schedule(use_stagger=False))
    one = torch.zeros(shape[0], shape[1], dtype=torch.float32, device=DEV)
    for b in (0, batch - 1):
        gemm2d(x[b], x_scales[b], w_t, w_scales, one)
        assert torch.equal(one, out[b])
