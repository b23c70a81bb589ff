"""GPU parity of the MXFP4 GEMM through the C ABI: golden fixtures and small
seeded cases against the exact oracle on every kernel variant and layout, the
edge cases the reference's tests touch (M = 1, K tails, ragged N, NaN scales),
and properties that hold at any size."""

import glob
import os

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import DEV, TILE_VARIANTS, assert_bf16_close, assert_close, assert_f32_close, run_gemm, to_gpu

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))

ALL_VARIANTS = dict(TILE_VARIANTS, skinny=_lib.VARIANT_SKINNY, naive=_lib.VARIANT_NAIVE, auto=_lib.VARIANT_AUTO)


@pytest.mark.parametrize("vname", sorted(ALL_VARIANTS))
@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(HERE, "golden", "g_*x*.npz"))),
                         ids=lambda p: os.path.basename(p)[:-4])
def test_golden_fixtures_every_variant(path, vname):
    g = np.load(path)
    x, xs, w_t, ws, ref = g["x"], g["x_scales"], g["w_t"], g["w_scales"], g["c_exact"]
    if vname == "skinny" and x.shape[0] > 64:
        pytest.skip("skinny kernel serves M <= 64")
    v = ALL_VARIANTS[vname]
    assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, variant=v), ref, "f32")
    assert_bf16_close(run_gemm(x, xs, w_t, ws, torch.bfloat16, variant=v), ref, "bf16")
    # shuffled scales (padded buffers) give the same numbers
    got = run_gemm(x, g["x_scales_shuffled"], w_t, g["w_scales_shuffled"], torch.float32, variant=v,
                   a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert_f32_close(got, ref, "shuffled scales")
    if g["w_t_preshuffled"].size:
        got = run_gemm(x, xs, g["w_t_preshuffled"], ws, torch.float32, variant=v, b_layout=_lib.B_PRESHUFFLE)
        assert_f32_close(got, ref, "preshuffled B")
    # without scratch the kernels read each layout directly; with MFMA32 scales
    # given by the caller they need no pre-pass
    assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, variant=v, workspace=False), ref, "direct row-major")
    got = run_gemm(x, g["x_scales_shuffled"], w_t, g["w_scales_shuffled"], torch.float32, variant=v,
                   a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE, workspace=False)
    assert_f32_close(got, ref, "direct shuffled")
    got = run_gemm(x, orc.mfma32_scale_layout(xs), w_t, orc.mfma32_scale_layout(ws), torch.float32, variant=v,
                   a_scale_layout=_lib.SCALE_MFMA32, b_scale_layout=_lib.SCALE_MFMA32, workspace=False)
    assert_f32_close(got, ref, "MFMA32 scales")
    got = run_gemm(x, orc.mfma32_scale_layout(xs), w_t, ws, torch.bfloat16, variant=v,
                   a_scale_layout=_lib.SCALE_MFMA32, workspace=False)
    assert_bf16_close(got, ref, "mixed scale layouts")


SMALL_SHAPES = [
    (256, 256, 256), (512, 384, 1024), (300, 200, 512), (129, 257, 768), (1, 1, 32), (2, 3, 64),
    (64, 64, 2048), (17, 1000, 1024), (1000, 17, 256), (255, 255, 8192), (4, 6, 224), (96, 130, 1664),
]


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("m,n,k", SMALL_SHAPES)
def test_auto_dispatch_small_shapes(m, n, k, out_dtype):
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + n + k, scale_lo=120, scale_hi=134)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    assert_close(run_gemm(x, xs, w_t, ws, out_dtype), ref, out_dtype, f"{m}x{n}x{k}")


@pytest.mark.parametrize("vname", sorted(TILE_VARIANTS))
@pytest.mark.parametrize("m,n,k", [(512, 512, 512), (300, 520, 1280), (1, 40, 256), (257, 33, 2304)])
def test_tile_variants_ragged_shapes(m, n, k, vname):
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=7 * m + n, scale_lo=110, scale_hi=140)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, variant=TILE_VARIANTS[vname]), ref, vname)


@pytest.mark.parametrize("m", [1, 5, 16, 17, 32, 48, 64])
@pytest.mark.parametrize("n,k", [(128, 1024), (1000, 4096), (48, 256), (30, 160)])
def test_skinny_kernel(m, n, k):
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m * 31 + n, scale_lo=120, scale_hi=134)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    assert_bf16_close(run_gemm(x, xs, w_t, ws, torch.bfloat16, variant=_lib.VARIANT_SKINNY), ref)
    assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, variant=_lib.VARIANT_SKINNY), ref)


@pytest.mark.parametrize("vname", ["t128x128_w2x2", "t256x256_w2x2", "skinny"])
@pytest.mark.parametrize("splits", [2, 4])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_split_k_equals_unsplit(vname, splits, out_dtype):
    m = 48 if vname == "skinny" else 384
    n, k = 640, 2048
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=splits, scale_lo=120, scale_hi=134)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    v = ALL_VARIANTS[vname]
    got = run_gemm(x, xs, w_t, ws, out_dtype, variant=v, split_k=splits)
    # f32 partials + one final rounding: the bf16 result stays within one ulp
    assert_close(got, ref, out_dtype, f"{vname} split {splits}")
    # C is overwritten, not accumulated into: a second call gives the same bits
    again = run_gemm(x, xs, w_t, ws, out_dtype, variant=v, split_k=splits)
    assert np.array_equal(got, again)


@pytest.mark.parametrize("splits", [3, 5, 6, 7, 8])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_split_k_part_counts(splits, out_dtype):
    """Every part count the library's own split can take (the sum over the parts has an unrolled form per count),
    on the 128x128 and 128x256 tiles, with an M x N that is and is not a multiple of four."""
    for m, n in ((200, 384), (131, 250)):
        k = splits * 512
        x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=splits, scale_lo=120, scale_hi=134)
        ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
        for v in (_lib.VARIANT_T128x128_W2x2, _lib.VARIANT_T128x256_W2x2):
            got = run_gemm(x, xs, w_t, ws, out_dtype, variant=v, split_k=splits)
            assert not np.isnan(got).any()
            assert_close(got, ref, out_dtype, f"{m}x{n} variant {v} split {splits}")


def test_split_k_auto_and_caller_workspace():
    m, n, k = 256, 256, 8192
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=3)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    need = wave_amd.workspace_bytes(m, n, k, split_k=0)
    assert need > 0                      # a 1-tile grid with long K: the library wants to split
    work = torch.empty(need, dtype=torch.uint8, device=DEV)
    assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, split_k=0, workspace=work), ref)
    with pytest.raises(ValueError, match="K per split"):
        run_gemm(x, xs, w_t, ws, torch.float32, split_k=3)


def test_exact_when_sums_fit_24_bits():
    """Scales 124..127: every product is a multiple of 2^-8 and the sums stay
    below 2^16, so the f32 result must equal the exact one bit for bit, on
    every kernel (any summation order)."""
    x, xs, w_t, ws = orc.make_inputs(320, 288, 1024, seed=9, scale_lo=124, scale_hi=127)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws).astype(np.float32)
    for vname, v in ALL_VARIANTS.items():
        if vname == "skinny":
            continue
        assert np.array_equal(run_gemm(x, xs, w_t, ws, torch.float32, variant=v), ref), vname
    assert np.array_equal(run_gemm(x[:64], xs[:64], w_t, ws, torch.float32, variant=_lib.VARIANT_SKINNY), ref[:64])


def test_one_hot_rows_read_back_dequantised_b_exactly():
    """A row with a single 1.0 at element e and scale 2^0 makes C[m, :] the
    dequantised column e of B: every value is representable, so it must match
    the bit-exact dequantiser exactly (nibble order, scale group, layout)."""
    n, k = 96, 512
    rng = np.random.default_rng(4)
    w_t = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    ws = rng.integers(100, 155, size=(n, k // 32), dtype=np.uint8)
    picks = [0, 1, 31, 32, 33, 255, 256, 257, 511]
    x = np.zeros((len(picks), k // 2), dtype=np.uint8)
    for r, e in enumerate(picks):
        x[r, e // 2] = 2 << (4 * (e & 1))          # code 2 = 1.0
    xs = np.full((len(picks), k // 32), 127, dtype=np.uint8)
    deq = orc.dequant_f32(w_t, ws)
    want = deq[:, picks].T.astype(np.float32)
    for v in (_lib.VARIANT_SKINNY, _lib.VARIANT_T128x128_W2x2, _lib.VARIANT_T256x256_W2x2):
        got = run_gemm(x, xs, w_t, ws, torch.float32, variant=v)
        assert np.array_equal(got, want), v


def test_nan_scale_poisons_its_row_and_column():
    x, xs, w_t, ws = orc.make_inputs(70, 90, 512, seed=5)
    xs[3, 2] = 255
    ws[40, 15] = 255
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    for v in (_lib.VARIANT_T128x128_W2x2, _lib.VARIANT_T256x256_W4x2, _lib.VARIANT_NAIVE):
        assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, variant=v), ref, str(v))
    assert_f32_close(run_gemm(x[:8], xs[:8], w_t, ws, torch.float32, variant=_lib.VARIANT_SKINNY), ref[:8])


def test_extreme_scales_zero_byte():
    """Scale byte 0 is 2^-127; paired with a large scale the product is an
    ordinary number and must not be flushed."""
    m, n, k = 32, 32, 256
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=6)
    xs[:] = 0
    ws[:] = 250
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    assert np.abs(ref).max() > 1.0
    for v in (_lib.VARIANT_T128x128_W2x2, _lib.VARIANT_SKINNY):
        assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, variant=v), ref, str(v))


def test_row_and_column_permutation_equivariance():
    """Permuting rows of A (with their scales) permutes rows of C bit for bit;
    same for rows of B and columns of C."""
    m, n, k = 512, 512, 1024
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=8, scale_lo=110, scale_hi=140)
    base = run_gemm(x, xs, w_t, ws, torch.float32)
    rng = np.random.default_rng(0)
    pm, pn = rng.permutation(m), rng.permutation(n)
    assert np.array_equal(run_gemm(x[pm], xs[pm], w_t, ws, torch.float32), base[pm])
    assert np.array_equal(run_gemm(x, xs, w_t[pn], ws[pn], torch.float32), base[:, pn])


def test_scale_shift_is_exact_power_of_two():
    """Adding 1 to every A scale byte doubles C exactly."""
    x, xs, w_t, ws = orc.make_inputs(200, 136, 768, seed=10, scale_lo=120, scale_hi=130)
    a = run_gemm(x, xs, w_t, ws, torch.float32)
    b = run_gemm(x, xs + 1, w_t, ws, torch.float32)
    assert np.array_equal(b, 2.0 * a)


def test_repeatable_and_poisoned_output():
    """Same inputs, same bits, on every call; the kernel overwrites whatever C held."""
    x, xs, w_t, ws = orc.make_inputs(700, 520, 2048, seed=11)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    outs = []
    for fill in (0.0, float("nan"), 1e30):
        out = torch.full((700, 520), fill, dtype=torch.float32, device=DEV)
        wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out)
        outs.append(out.cpu().numpy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_non_contiguous_inputs_and_side_stream():
    """Non-contiguous operands are copied, not rejected; work goes to the
    current stream without a sync (reference launch semantics)."""
    m, n, k = 128, 192, 512
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=12)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    w_view = gw.T.contiguous().T           # [N, K/2] values, column-major storage
    assert not w_view.is_contiguous()
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert wave_amd.mxfp4_gemm(gx, gxs, w_view, gws, out) is None
    side.synchronize()
    assert_f32_close(out.cpu().numpy(), ref)


def test_bad_arguments_raise():
    x, xs, w_t, ws = to_gpu(*orc.make_inputs(64, 64, 256, seed=13))
    out = torch.empty(64, 64, dtype=torch.float32, device=DEV)
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(x, xs, w_t[:, :64], ws, out)            # K mismatch
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(x, xs[:, :4], w_t, ws, out)             # scale shape
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(x, xs, w_t, ws, out.to(torch.float16))  # out dtype
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(x, xs, w_t, ws, out[:32])               # out shape
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(x.float(), xs, w_t, ws, out)            # operand dtype


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("vname", ["t256x256_w2x2", "t256x256_w4x2"])
@pytest.mark.parametrize("shape", [(4352, 4352, 768), (4608, 4352, 1024)], ids=lambda s: "x".join(map(str, s)))
def test_persistent_path_more_tiles_than_cus(shape, vname, out_dtype):
    """More 256x256 tiles than workgroups: some workgroups compute two or three
    tiles in a row, with the operand stream running across the tile boundary
    and the C stores of one tile in flight under the next (scales reach the
    kernel in MFMA32 order through the scratch pre-pass)."""
    m, n, k = shape
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=118, scale_hi=136)
    rng = np.random.default_rng(7)
    rows = np.unique(np.concatenate([rng.integers(0, m, size=40), [0, 255, 256, m - 257, m - 256, m - 1]]))
    ref_rows = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    naive = run_gemm(x, xs, w_t, ws, torch.float32, variant=_lib.VARIANT_NAIVE)
    assert_f32_close(naive[rows], ref_rows, "naive vs oracle rows")
    v = TILE_VARIANTS[vname]
    got = run_gemm(x, xs, w_t, ws, out_dtype, variant=v)
    assert_close(got[rows], ref_rows, out_dtype, "persistent vs oracle rows")
    assert_close(got, naive, out_dtype, "persistent vs naive, all elements")
    # preshuffled B and caller-provided MFMA32 scales take the same path
    gx, gw = to_gpu(x, w_t)
    gwp = wave_amd.b_preshuffle(gw).cpu().numpy()
    got = run_gemm(x, orc.mfma32_scale_layout(xs), gwp, orc.mfma32_scale_layout(ws), out_dtype, variant=v,
                   a_scale_layout=_lib.SCALE_MFMA32, b_scale_layout=_lib.SCALE_MFMA32, b_layout=_lib.B_PRESHUFFLE,
                   workspace=False)
    assert_close(got, naive, out_dtype, "persistent, preshuffled B, MFMA32 scales")
    # and twice in a row into the same output (stale stores must not land late)
    got2 = run_gemm(x, xs, w_t, ws, out_dtype, variant=v)
    assert np.array_equal(got2, run_gemm(x, xs, w_t, ws, out_dtype, variant=v))


@pytest.mark.parametrize("m,n", [(3, 69648), (16, 36864), (33, 40976), (64, 36880)])
@pytest.mark.parametrize("layout", ["row_major", "mfma32_preshuffled"])
def test_streaming_kernel_many_tiles_per_workgroup(m, n, layout):
    """K = 8192 decode shapes whose N gives every workgroup more 16-row tiles
    of B than it can hold finished sums for (8), so that C is also written in
    the middle of the stream, with a ragged last tile and an uneven split of
    tiles over workgroups."""
    k = 8192
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=n + m, scale_lo=120, scale_hi=134)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    if layout == "row_major":
        got = run_gemm(x, xs, w_t, ws, torch.bfloat16, variant=_lib.VARIANT_SKINNY)
        assert_bf16_close(got, ref, "row-major")
        got = run_gemm(x, xs, w_t, ws, torch.float32, variant=_lib.VARIANT_SKINNY)
        assert_f32_close(got, ref, "row-major f32")
    else:
        (gw,) = to_gpu(w_t)
        gwp = wave_amd.b_preshuffle(gw).cpu().numpy()
        got = run_gemm(x, orc.mfma32_scale_layout(xs), gwp, orc.mfma32_scale_layout(ws), torch.float32,
                       variant=_lib.VARIANT_SKINNY, a_scale_layout=_lib.SCALE_MFMA32,
                       b_scale_layout=_lib.SCALE_MFMA32, b_layout=_lib.B_PRESHUFFLE)
        assert_f32_close(got, ref, "MFMA32 scales, preshuffled B")
        got = run_gemm(x, orc.e8m0_shuffle_padded(xs)[:(m + 31) // 32 * 32], w_t,
                       orc.e8m0_shuffle_padded(ws)[:(n + 31) // 32 * 32], torch.bfloat16,
                       variant=_lib.VARIANT_SKINNY, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                       b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
        assert_bf16_close(got, ref, "shuffled scales")


@pytest.mark.parametrize("k", [1024, 2048, 3072, 4096, 5120, 7168])
@pytest.mark.parametrize("m", [5, 17])
def test_streaming_kernel_fewer_k_tiles_per_wave(m, k):
    """Decode shapes whose K gives each of the four waves 1..7 K tiles instead
    of 8 (odd counts start odd waves on an odd K tile), in every scale layout;
    NaN scales at the very end of a row must poison exactly their row/column,
    also where lanes past the wave's range re-fetch that end."""
    n = 8208
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=k + m, scale_lo=120, scale_hi=134)
    ws[3, -1] = 255
    ws[n - 1, -1] = 255
    xs[m - 1, -1] = 255
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    assert np.isnan(ref[:, 3]).all() and np.isnan(ref[m - 1]).all() and not np.isnan(ref[0, 0])
    got = run_gemm(x, xs, w_t, ws, torch.float32, variant=_lib.VARIANT_SKINNY)
    assert_f32_close(got, ref, "row-major")
    got = run_gemm(x, xs, w_t, ws, torch.bfloat16)
    assert_bf16_close(got, ref, "row-major, auto, bf16")
    (gw,) = to_gpu(w_t)
    gwp = wave_amd.b_preshuffle(gw).cpu().numpy()
    got = run_gemm(x, orc.mfma32_scale_layout(xs), gwp, orc.mfma32_scale_layout(ws), torch.float32,
                   variant=_lib.VARIANT_SKINNY, a_scale_layout=_lib.SCALE_MFMA32,
                   b_scale_layout=_lib.SCALE_MFMA32, b_layout=_lib.B_PRESHUFFLE)
    assert_f32_close(got, ref, "MFMA32 scales, preshuffled B")
    got = run_gemm(x, orc.e8m0_shuffle_padded(xs)[:(m + 31) // 32 * 32], w_t,
                   orc.e8m0_shuffle_padded(ws)[:(n + 31) // 32 * 32], torch.float32,
                   variant=_lib.VARIANT_SKINNY, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                   b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert_f32_close(got, ref, "shuffled scales")


@pytest.mark.parametrize("vname,m,split", [("auto", 16, 1), ("auto", 200, 1), ("t256x256_w2x2", 300, 1),
                                           ("t128x128_w2x2", 384, 2), ("naive", 33, 1), ("auto", 4352, 1)])
def test_one_scale_per_row_of_a(vname, m, split):
    """a_scale [M], held for every 32-group of the row (the reference's
    broadcast-scale kernel): same bits as the GEMM on the spread-out matrix, and
    parity with the oracle on it."""
    n, k = (4352, 768) if m > 1000 else (272, 2048)
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m, scale_lo=118, scale_hi=136)
    per_row = np.ascontiguousarray(xs[:, 0])
    spread = np.repeat(per_row[:, None], k // 32, axis=1)
    v = ALL_VARIANTS[vname]
    got = run_gemm(x, per_row, w_t, ws, torch.float32, variant=v, split_k=split)
    same = run_gemm(x, spread, w_t, ws, torch.float32, variant=v, split_k=split)
    assert np.array_equal(got, same)
    if m <= 1000:
        assert_f32_close(got, c_oracle.scaled_gemm_exact(x, w_t, spread, ws), vname)
    # it needs the scratch buffer; without one the call is refused, nothing runs
    gx, gs, gw, gws = to_gpu(x, per_row, w_t, ws)
    out = torch.zeros(m, n, dtype=torch.float32, device=DEV)
    with pytest.raises(ValueError, match="workspace"):
        wave_amd.mxfp4_gemm(gx, gs, gw, gws, out, variant=v, workspace=False)
    assert not bool(out.any())


@pytest.mark.parametrize("batch,m,n,k", [(4, 96, 160, 512), (8, 1, 16384, 1664), (3, 16, 272, 8192)])
def test_batched_a_with_shared_b(batch, m, n, k):
    x, xs, w_t, ws = orc.make_inputs(batch * m, n, k, seed=batch + m)
    gx, gxs, gw, gws = to_gpu(x.reshape(batch, m, k // 2), xs.reshape(batch, m, k // 32), w_t, ws)
    out = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out)
    torch.cuda.synchronize()
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    assert_f32_close(out.cpu().numpy().reshape(batch * m, n), ref)
    with pytest.raises(ValueError, match="out"):
        wave_amd.mxfp4_gemm(gx, gxs, gw, gws, torch.empty(batch * m, n, dtype=torch.float32, device=DEV))


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("vname", ["t256x256_w2x2", "t256x256_w4x2"])
@pytest.mark.parametrize("m", [4352 - 255, 4352 - 3, 4097])
def test_persistent_path_ragged_m(m, vname, out_dtype):
    """More tiles than CUs with a last tile row that runs past M: the rows past M
    are read as zeros and never stored (a canary behind C stays intact)."""
    n, k = 4352, 768
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m, scale_lo=120, scale_hi=134)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    buf = torch.full(((m + 300) * n,), 7.0, dtype=out_dtype, device=DEV)
    out = buf[: m * n].view(m, n)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, variant=ALL_VARIANTS[vname])
    torch.cuda.synchronize()
    assert bool((buf[m * n:] == 7.0).all())
    rows = np.r_[0:64, m - 300:m]              # the oracle on the first rows and on the last two tile rows
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    assert_close(out.float().cpu().numpy()[rows], ref, out_dtype, f"{vname} M={m}")
    # the one-tile-per-workgroup kernel (no scratch: scales read as given) agrees on every element
    other = torch.empty_like(out)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, other, variant=ALL_VARIANTS[vname], workspace=False)
    torch.cuda.synchronize()
    diff = (out.float() - other.float()).abs().max().item()
    assert diff <= (2e-6 if out_dtype == torch.float32 else 2.0 ** -7) * out.float().abs().max().item()


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("vname", sorted(TILE_VARIANTS))
@pytest.mark.parametrize("m,n,k", [(300, 520, 1248), (512, 512, 800), (257, 264, 288), (128, 128, 32 + 256 * 3)])
def test_partial_last_k_tile_every_tile_kernel(m, n, k, vname, out_dtype):
    """K % 256 != 0: with scratch the scales are re-laid out and the lanes past the end of K fetch zeros from beyond
    the buffer descriptor (any tile kernel); without scratch the generic 128x128 kernel runs.  Both against the
    oracle.  A NaN scale in the last group that exists must still poison its row."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=k + m, scale_lo=118, scale_hi=136)
    xs[3, -1] = 255
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    v = ALL_VARIANTS[vname]
    assert_close(run_gemm(x, xs, w_t, ws, out_dtype, variant=v), ref, out_dtype, f"{vname} with scratch")
    assert_close(run_gemm(x, xs, w_t, ws, out_dtype, variant=v, workspace=False), ref, out_dtype, f"{vname} without")


def test_partial_last_k_tile_full_size_sampled_rows():
    """8192 x 8192 x 16000 (a shape of the reference's benchmark list,
    wave_lang/kernel/wave/perf/mxfp4_shapes_macrotiles.csv): sampled rows against the oracle."""
    m, n, k = 8192, 8192, 16000
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=16)
    rows = np.r_[0:8, 4093:4099, 8184:8192]
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    got = run_gemm(x, xs, w_t, ws, torch.bfloat16)
    assert_bf16_close(got[rows], ref)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("vname", ["t256x256_w2x2", "t256x256_w4x2"])
@pytest.mark.parametrize("k", [1024 + 128, 1024 + 32, 2048 - 32])
def test_persistent_path_partial_last_k_tile(k, vname, out_dtype):
    """More tiles than CUs and K % 256 != 0 (128 is the remainder of K = 16000, the K of the reference's
    benchmark shapes); ragged M on top.  A NaN scale in the last existing group must poison its row and column."""
    m, n = 4352 - 100, 4352
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=k, scale_lo=120, scale_hi=134)
    xs[7, -1] = 255
    ws[9, -1] = 255
    rows = np.r_[0:40, m - 200:m]
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    got = run_gemm(x, xs, w_t, ws, out_dtype, variant=ALL_VARIANTS[vname])
    assert_close(got[rows], ref, out_dtype, f"{vname} K={k}")
    assert np.isnan(got[7]).all() and np.isnan(got[:, 9]).all() and not np.isnan(np.delete(np.delete(got, 7, 0), 9, 1)).any()


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("m,n,k", [(4608, 4096, 4096 + 128), (4608 - 70, 4096, 2304), (2560, 8192, 1024 + 64 * 32)])
def test_persistent_path_last_round_cut_along_k(m, n, k, out_dtype):
    """288 or 320 tiles on 256 CUs: the tiles of the last round are cut along K over the idle workgroups and
    summed afterwards (with and without a partial last K tile, ragged M).  Two rows of every tile row against
    the oracle, and every element against the one-tile-per-workgroup kernel."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=120, scale_hi=134)
    rows = np.array(sorted({min(m - 1, b * 256 + o) for b in range((m + 255) // 256) for o in (3, 250)}))
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    buf = torch.full(((m + 64) * n,), 7.0, dtype=out_dtype, device=DEV)
    out = buf[: m * n].view(m, n)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, variant=_lib.VARIANT_T256x256_W4x2)
    torch.cuda.synchronize()
    assert bool((buf[m * n:] == 7.0).all())
    assert_close(out.float().cpu().numpy()[rows], ref, out_dtype, f"{m}x{n}x{k}")
    other = torch.empty_like(out)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, other, variant=_lib.VARIANT_T128x128_W2x2)
    torch.cuda.synchronize()
    diff = (out.float() - other.float()).abs().max().item()
    assert diff <= (4e-6 if out_dtype == torch.float32 else 2.0 ** -7) * out.float().abs().max().item()


@pytest.mark.parametrize("vname", ["t128x128_w2x2", "t256x256_w4x2"])
@pytest.mark.parametrize("m,n,k", [(300, 528, 1248 - 32), (4352 - 100, 4352, 1024 + 128)])
def test_partial_last_k_tile_preshuffled_b_and_shuffled_scales(m, n, k, vname):
    """The reference's fastest templates (preshuffled B, e8m0_shuffle scales) at K % 256 != 0 (K % 64 == 0 as
    b_preshuffle needs): same bits as the row-major operands on the same kernel."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=n + k, scale_lo=120, scale_hi=134)
    v = ALL_VARIANTS[vname]
    plain = run_gemm(x, xs, w_t, ws, torch.float32, variant=v)
    rows = np.r_[0:32, m - 40:m]
    assert_f32_close(plain[rows], c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows), vname)
    pre = run_gemm(x, orc.e8m0_shuffle_padded(xs)[: (m + 31) // 32 * 32], orc.b_preshuffle(w_t),
                   orc.e8m0_shuffle_padded(ws)[: (n + 31) // 32 * 32], torch.float32, variant=v,
                   a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                   b_layout=_lib.B_PRESHUFFLE)
    assert np.array_equal(pre, plain)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("m,n,k", [(1024, 2048, 16000), (1000, 1920, 48 * 256 + 256), (512, 640, 9 * 256),
                                   (384, 512, 11 * 256 + 64)])
def test_automatic_split_with_uneven_parts(m, n, k, out_dtype):
    """Few tiles and a long K whose tile count the split count does not divide (63 K tiles in 2 parts, 9 in 8 ...):
    the last part is shorter and owns the partial last K tile.  Sampled rows against the oracle."""
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=m + k, scale_lo=122, scale_hi=132)
    rows = np.r_[0:6, m // 2 - 3:m // 2 + 3, m - 6:m]
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    got = run_gemm(x, xs, w_t, ws, out_dtype)
    assert not np.isnan(got).any()
    assert_close(got[rows], ref, out_dtype, f"{m}x{n}x{k}")


@pytest.mark.parametrize("k_tiles", [1, 2, 7, 16, 17])
def test_row_major_scales_without_scratch_short_and_long_k(k_tiles):
    """Without scratch the 128x128 kernel copies the row-major scale rows of its tile into LDS when the workgroup
    has at most 16 K tiles and reads them from global memory per K tile otherwise; ragged M and N (rows past the
    tensors are clamped), odd K tile counts (the LDS row pitch depends on their parity)."""
    m, n, k = 300, 250, 256 * k_tiles
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=k_tiles, scale_lo=110, scale_hi=140)
    xs[5, 0] = 255
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    got = run_gemm(x, xs, w_t, ws, torch.float32, variant=_lib.VARIANT_T128x128_W2x2, workspace=False)
    assert np.isnan(got[5]).all() and not np.isnan(np.delete(got, 5, 0)).any()
    assert_f32_close(np.delete(got, 5, 0), np.delete(ref, 5, 0), f"{k_tiles} K tiles")


def test_repeated_calls_with_one_signature():
    """The wrapper checks a signature (shapes, types, device, options) once and then only contiguity: later calls
    with new contents, a non-contiguous operand of the same shape, and other options on the same tensors must all
    give their own right answers."""
    m, n, k = 300, 260, 1024
    outs = []
    for seed in (1, 2, 3):
        x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=seed, scale_lo=120, scale_hi=134)
        ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
        assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32), ref, f"seed {seed}")
        outs.append(ref)
    assert not np.array_equal(outs[0], outs[1])
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    wide = torch.zeros(n, k, dtype=torch.uint8, device=DEV)
    wide[:, ::2] = gw
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, wide[:, ::2], gws, out)          # same shape, strided: copied, not misread
    assert_f32_close(out.cpu().numpy(), ref, "strided w_t")
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, split_k=2)          # same tensors, another option
    assert_f32_close(out.cpu().numpy(), ref, "split_k=2")
    bf = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, bf)                      # same shapes, another output type
    assert_bf16_close(bf.float().cpu().numpy(), ref, "bf16 out")
    with pytest.raises(ValueError):
        wave_amd.mxfp4_gemm(gx, gxs, gw, gws, torch.empty(m, n, dtype=torch.float16, device=DEV))
