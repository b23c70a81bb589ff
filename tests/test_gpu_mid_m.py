"""GPU: the mid-M kernel (variant 8: 16 < M <= 256 against a wide B from HBM; the reference runs such shapes
through its generic tile kernel, tests/kernel/wave_gemm_mxfp_test.py:291-339) against the exact oracle: every row
block count, ragged M, N that is no multiple of the strip width (strips of 16 to 32 columns per wave), K with a
partial group of four K tiles, both output types, both B layouts, row-major and MFMA32 scales per operand,
e8m0_shuffle scales read in place, NaN scales, and the library's own choice of it at the decode shapes."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, assert_close, to_gpu

pytestmark = pytest.mark.gpu
V = _lib.VARIANT_MID_M
RM, SH, M32 = _lib.SCALE_ROW_MAJOR, _lib.SCALE_E8M0_SHUFFLE, _lib.SCALE_MFMA32


def run(x, xs, w, ws, dt, la=RM, lb=RM, pre=False, **kw):
    m, n, k = x.shape[0], w.shape[0], x.shape[1] * 2
    gx, gxs, gw, gws = to_gpu(x, xs, w, ws)
    if pre:
        gw = wave_amd.b_preshuffle(gw)
    if la != RM:
        gxs = wave_amd.scale_convert(gxs, m, k // 32, RM, la)
    if lb != RM:
        gws = wave_amd.scale_convert(gws, n, k // 32, RM, lb)
    out = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, a_scale_layout=la, b_scale_layout=lb,
                        b_layout=_lib.B_PRESHUFFLE if pre else _lib.B_ROW_MAJOR, **kw)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pre", [False, True])
@pytest.mark.parametrize("m,n,k", [(65, 128, 1024), (128, 256, 2048), (17, 96, 1024), (200, 4096, 2048),
                                   (256, 640, 1280), (33, 160, 4096), (7, 16, 1024), (192, 1008, 1536)])
def test_mid_small_shapes_whole_oracle(m, n, k, pre, dt):
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=112, scale_hi=140)
    ref = c_oracle.scaled_gemm_exact(x, w, xs, ws)
    assert_close(run(x, xs, w, ws, dt, pre=pre, variant=V, split_k=1), ref, dt, f"{m}x{n}x{k}")


@pytest.mark.parametrize("la,lb", [(RM, RM), (M32, M32), (RM, M32), (M32, RM), (SH, SH), (SH, RM)])
@pytest.mark.parametrize("m,n,k", [(100, 28676, 1280), (130, 20000, 1536), (250, 57344, 1024), (64, 12292, 1024)])
def test_mid_wide_n_strip_widths_and_scale_layouts(m, n, k, la, lb):
    """Wide N: the strip per wave is narrower than 32 columns for row-major B scales (28676 columns on 256 CUs:
    29 -> 32 wide strips no longer fit one round, 20000: 20 columns), N ends inside a strip, and the row-major
    and MFMA32 scale paths must give the same bits (the products and their order do not depend on the layout)."""
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=n + k, scale_lo=100, scale_hi=154)
    c = run(x, xs, w, ws, torch.float32, la=la, lb=lb, pre=(n % 16 == 0), variant=V, split_k=1)
    assert_close(c, c_oracle.scaled_gemm_exact(x, w, xs, ws), torch.float32, f"{m}x{n}x{k} {la}/{lb}")
    if (la, lb) != (RM, RM):
        assert np.array_equal(c, run(x, xs, w, ws, torch.float32, variant=V, split_k=1))


@pytest.mark.parametrize("la,lb", [(RM, RM), (M32, M32), (RM, M32), (M32, RM)])
@pytest.mark.parametrize("m,n,k", [(20, 2048, 2048), (32, 4100, 4096), (100, 3000, 2048), (256, 1500, 4096), (64, 5120, 6144)])
def test_mid_rotated_start_in_k(m, n, k, la, lb):
    """K in whole groups of 8 K tiles: the workgroups start at different K tiles (workgroup 8 i + x at tile i) and
    walk around the end of K, each through the scale groups of 4 and 8 K tiles from the middle of one on; enough
    strips that starts 0 .. 7 and beyond occur, every scale layout pair, the 32-row block shape (M <= 32) too."""
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + n, scale_lo=104, scale_hi=150)
    c = run(x, xs, w, ws, torch.float32, la=la, lb=lb, pre=(n % 16 == 0 and lb == RM), variant=V, split_k=1)
    assert_close(c, c_oracle.scaled_gemm_exact(x, w, xs, ws), torch.float32, f"{m}x{n}x{k} {la}/{lb}")


@pytest.mark.parametrize("m,n,k", [(20, 2048, 2048), (100, 3000, 2048), (256, 1504, 4096), (64, 28676, 1024), (33, 160, 1280)])
@pytest.mark.parametrize("la", [RM, M32, SH])
def test_mid_reads_shuffled_b_scales_in_place(m, n, k, la):
    """B's scales in e8m0_shuffle order (the reference's format for static weights, mxfp_utils.py:113-128), A's in
    any of the three, without scratch, so that no pass can re-lay them out: the kernel reads the blocks as they
    are; the bits of the MFMA32 path (the same strips, the same order of the sums)."""
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m * 7 + n, scale_lo=100, scale_hi=154)
    c = run(x, xs, w, ws, torch.float32, la=la, lb=SH, variant=V, split_k=1, workspace=False)
    assert_close(c, c_oracle.scaled_gemm_exact(x, w, xs, ws), torch.float32, f"{m}x{n}x{k} {la}/shuffle")
    assert np.array_equal(c, run(x, xs, w, ws, torch.float32, la=M32, lb=M32, variant=V, split_k=1, workspace=False))


@pytest.mark.parametrize("lb", [RM, M32])
@pytest.mark.parametrize("m,n,k", [(1, 1024, 1024), (31, 640, 2304), (130, 2048, 1536), (200, 700, 2048), (256, 28672, 1024)])
def test_mid_reads_shuffled_a_scales_in_place(m, n, k, lb):
    """A's scales in e8m0_shuffle order (what the quantiser writes for the reference's preshuffled-scale kernels)
    against B's row-major and MFMA32 ones, without scratch; M that ends inside a 32-row block of the layout."""
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m * 5 + k, scale_lo=100, scale_hi=154)
    c = run(x, xs, w, ws, torch.float32, la=SH, lb=lb, variant=V, split_k=1, workspace=False)
    cols = np.unique(np.concatenate([np.arange(0, n, max(1, n // 600)), [n - 1]]))
    assert_close(c[:, cols], c_oracle.scaled_gemm_exact(x, w[cols], xs, ws[cols]), torch.float32, f"{m}x{n}x{k} shuffle/{lb}")
    assert np.array_equal(c, run(x, xs, w, ws, torch.float32, la=M32, lb=lb, variant=V, split_k=1, workspace=False))


@pytest.mark.parametrize("lb", [RM, M32, SH])
@pytest.mark.parametrize("m,n,k", [(24, 36864, 2048), (1, 40004, 1024), (32, 33000, 1280)])
def test_mid_more_strips_than_cus(m, n, k, lb):
    """Up to 32 rows against more 128-column strips than the GPU has CUs: the shallow rings with two workgroups per
    CU; sampled columns of every strip region against the oracle, AUTO the same bits."""
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=n, scale_lo=110, scale_hi=144)
    c = run(x, xs, w, ws, torch.float32, lb=lb, variant=V, split_k=1)
    cols = np.unique(np.concatenate([np.arange(0, n, 97), np.arange(n - 130, n)]))
    ref = c_oracle.scaled_gemm_exact(x, w[cols], xs, ws[cols])
    assert_close(c[:, cols], ref, torch.float32, f"{m}x{n}x{k} {lb}")
    assert not np.isnan(c).any()
    assert np.array_equal(run(x, xs, w, ws, torch.float32, lb=lb), c)


@pytest.mark.parametrize("m", [17, 32, 48, 64, 128, 256])
def test_mid_decode_shapes_and_auto_choice(m):
    """cfg3's N and K at M = 17 .. 256, bf16 out: sampled rows against the oracle (all rows up to 64), all elements
    against the tile kernel; for M the library takes the kernel by itself, AUTO gives the same bits."""
    n, k = 28672, 8192
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=2, scale_lo=120, scale_hi=134)
    c = run(x, xs, w, ws, torch.bfloat16, variant=V, split_k=1)
    rows = np.arange(m) if m <= 64 else np.unique(np.concatenate([np.arange(0, m, 5), [m - 1]]))
    assert_close(c[rows], c_oracle.scaled_gemm_exact(x, w, xs, ws, rows=rows), torch.bfloat16, "rows vs oracle")
    other = run(x, xs, w, ws, torch.float32, variant=_lib.VARIANT_T128x128_W2x2, split_k=1)
    assert_close(c, other.astype(np.float64), torch.bfloat16, "all elements vs the tile kernel")
    assert np.array_equal(run(x, xs, w, ws, torch.bfloat16), c)


def test_mid_nan_scale_poisons_its_row_and_column():
    m, n, k = 96, 640, 2048
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=5, scale_lo=120, scale_hi=134)
    xs[70, 17] = 255
    ws[77, 63] = 255
    c = run(x, xs, w, ws, torch.float32, variant=V, split_k=1)
    assert np.isnan(c[70]).all() and np.isnan(c[:, 77]).all()
    assert_close(c, c_oracle.scaled_gemm_exact(x, w, xs, ws), torch.float32, "NaN scales")


def test_mid_rejects_what_it_does_not_take():
    x, xs, w, ws = orc.make_inputs(300, 256, 1024, seed=1)
    with pytest.raises((RuntimeError, ValueError)):
        run(x, xs, w, ws, torch.float32, variant=V, split_k=1)          # M > 256
    x, xs, w, ws = orc.make_inputs(64, 256, 512, seed=1)
    with pytest.raises((RuntimeError, ValueError)):
        run(x, xs, w, ws, torch.float32, variant=V, split_k=1)          # fewer than 4 K tiles
    x, xs, w, ws = orc.make_inputs(64, 256, 2048, seed=1)
    with pytest.raises((RuntimeError, ValueError)):
        run(x, xs, w, ws, torch.float32, variant=V, split_k=2)          # it takes whole K ranges


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(16, 5760, 2880), (64, 2880, 2880), (1, 4096, 1056), (200, 4100, 2848),
                                   (256, 640, 1312), (33, 8192, 4000), (130, 1008, 2080)])
def test_mid_partial_last_k_tile(m, n, k, dt):
    """K in whole scale groups of 32 but not in whole K tiles of 256 (2880: the hidden size of gpt-oss): the kernel
    walks ceil(K / 256) K tiles, and what the last one brings in from past the end of K is multiplied with the zero
    padding of MFMA32-ordered scales (2^-127 each), which vanishes in f32.  By name with the scales handed over in
    MFMA32 order, with row-major ones re-laid in scratch, with B preshuffled, and the library's own choice; without
    scratch and row-major scales the kernel is refused by name and the library's choice takes another one.  Every
    element against the exact oracle, last rows and columns included."""
    x, xs, w, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=112, scale_hi=140)
    ref = c_oracle.scaled_gemm_exact(x, w, xs, ws)
    assert_close(run(x, xs, w, ws, dt, la=M32, lb=M32, variant=V, split_k=1), ref, dt, f"{m}x{n}x{k} MFMA32 scales")
    assert_close(run(x, xs, w, ws, dt, variant=V, split_k=1), ref, dt, f"{m}x{n}x{k} row-major scales, scratch")
    if n % 16 == 0 and k % 64 == 0:
        assert_close(run(x, xs, w, ws, dt, la=M32, lb=M32, pre=True, variant=V, split_k=1), ref, dt, f"{m}x{n}x{k} preshuffled B")
    assert_close(run(x, xs, w, ws, dt), ref, dt, f"{m}x{n}x{k} library's choice")
    assert_close(run(x, xs, w, ws, dt, la=M32, lb=M32), ref, dt, f"{m}x{n}x{k} library's choice, MFMA32 scales")
    assert_close(run(x, xs, w, ws, dt, workspace=False), ref, dt, f"{m}x{n}x{k} library's choice without scratch")
    with pytest.raises((RuntimeError, ValueError)):
        run(x, xs, w, ws, dt, variant=V, split_k=1, workspace=False)
