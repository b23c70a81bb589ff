"""GPU: the grouped GEMM at a small batch (a few rows per expert: the decode step of a mixture of experts, the
per-expert loop of tests/kernel/moe_test.py:175-246 at serving sizes) through the mid-M kernel, one workgroup per
(expert, strip of columns), against the exact oracle applied per group: ragged and empty groups, groups of more rows
than one block, N that ends inside a strip, row-major and MFMA32 expert scales, activation scales row-major or in
MFMA32 order, preshuffled expert weights, both
output types, rows past the last offset left alone, and the library's own choice of it."""

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
RM, M32, SH = _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32, _lib.SCALE_E8M0_SHUFFLE


def inputs(e, n, k, rows, seed, force_empty=(), lo=118, hi=136):
    off = orc.make_group_offsets(e, rows, seed, force_empty=force_empty)
    x, xs, _, _ = orc.make_inputs(rows, 1, k, seed, scale_lo=lo, scale_hi=hi)
    rng = np.random.default_rng(seed + 100)
    w = rng.integers(0, 256, size=(e, n, k // 2), dtype=np.uint8)
    ws = rng.integers(lo, hi + 1, size=(e, n, k // 32), dtype=np.uint8)
    return x, xs, w, ws, off


def reference(x, xs, w, ws, off):
    out = np.full((x.shape[0], w.shape[1]), np.nan)
    for g in range(len(off) - 1):
        a, b = int(off[g]), int(off[g + 1])
        if b > a:
            out[a:b] = c_oracle.scaled_gemm_exact(x[a:b], w[g], xs[a:b], ws[g])
    return out


def run(x, xs, w, ws, off, dt, lb=RM, pre=False, la=RM, **kw):
    e, n, k = w.shape[0], w.shape[1], x.shape[1] * 2
    gx, gxs, gw, gws, goff = to_gpu(x, xs, w, ws, off)
    if la != RM:   # one tensor over all rows: its 32-row blocks straddle the groups
        gxs = wave_amd.scale_convert(gxs, x.shape[0], k // 32, RM, la)
        kw["a_scale_layout"] = la
    if pre:
        gw = torch.stack([wave_amd.b_preshuffle(gw[g]) for g in range(e)])
    if lb != RM:
        gws = torch.stack([wave_amd.scale_convert(gws[g], n, k // 32, RM, lb) for g in range(e)])
    out = torch.full((x.shape[0], n), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out, b_scale_layout=lb,
                                b_layout=_lib.B_PRESHUFFLE if pre else _lib.B_ROW_MAJOR, **kw)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def check(c, ref, dt, what):
    done = ~np.isnan(ref)
    assert np.isnan(c[~done]).all(), f"{what}: rows of no group were written"
    assert_close(c[done.all(axis=1)], ref[done.all(axis=1)], dt, what)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lb,pre", [(RM, False), (M32, False), (RM, True), (M32, True), (SH, False), (SH, True)])
@pytest.mark.parametrize("e,n,k,rows", [(8, 160, 1024, 40), (5, 1008, 1280, 333), (16, 96, 2048, 16), (3, 4096, 1024, 700),
                                        (40, 1024, 2048, 300)])
def test_grouped_mid_ragged_groups(e, n, k, rows, lb, pre, dt):
    """Uneven groups (333 rows over 5 experts and 700 over 3: groups of more rows than a block, taken block by
    block; 16 rows over 16 experts: groups of one row and none; 40 experts x 8 strips: more strips than CUs, the
    shallow rings with two workgroups per CU, K walked from a rotated start)."""
    x, xs, w, ws, off = inputs(e, n, k, rows, seed=e + rows)
    c = run(x, xs, w, ws, off, dt, lb=lb, pre=pre, variant=V)
    check(c, reference(x, xs, w, ws, off), dt, f"E={e} {rows}x{n}x{k}")


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lb,pre", [(RM, False), (M32, False), (M32, True), (SH, False)])
@pytest.mark.parametrize("e,n,k,rows", [(8, 160, 1024, 40), (5, 1008, 1280, 333), (16, 96, 2048, 16), (3, 4096, 1024, 700),
                                        (40, 1024, 2048, 300), (8, 512, 1024, 8 * 200)])
def test_grouped_mid_activation_scales_in_mfma32_order(e, n, k, rows, lb, pre, dt):
    """The activations' scales as the gathered quantiser writes them for the tile kernels: one [rows, K/32] tensor in
    MFMA32 order whose 32-row blocks ignore the group borders, so a group's block of rows starts at any row of a
    scale block and reads one block more than its rows span.  Same groups as above (one-row groups, groups of more
    rows than the block, more strips than CUs) and 200 rows per expert on average (the 192-row block: the
    256-row block has no room for the extra scale block); every block height is reached through the average."""
    x, xs, w, ws, off = inputs(e, n, k, rows, seed=e + rows + 1)
    c = run(x, xs, w, ws, off, dt, lb=lb, pre=pre, la=M32, variant=V)
    check(c, reference(x, xs, w, ws, off), dt, f"E={e} {rows}x{n}x{k} A scales MFMA32")


def test_grouped_mid_mfma32_activation_scales_nan_stays_in_its_row():
    """A NaN scale (byte 255) in the last row of one group and the first row of the next: exactly those two rows of C
    are NaN, although both groups' blocks read the scale block the rows share."""
    e, n, k, rows = 4, 256, 1024, 100
    x, xs, w, ws, off = inputs(e, n, k, rows, seed=9, lo=124, hi=130)
    r = int(off[2])
    assert 0 < r < rows and off[1] < off[2] < off[3]
    xs[r - 1, 5] = 255
    xs[r, 17] = 255
    c = run(x, xs, w, ws, off, torch.float32, la=M32, variant=V)
    nan_rows = np.isnan(c).all(axis=1)
    assert np.array_equal(np.nonzero(nan_rows)[0], [r - 1, r])
    assert not np.isnan(np.delete(c, [r - 1, r], axis=0)).any()


@pytest.mark.parametrize("force_empty", [(0,), (3, 4), (7,), (0, 1, 2, 3, 4, 5, 6)])
def test_grouped_mid_empty_groups_and_rows_past_the_last_offset(force_empty):
    e, n, k = 8, 640, 1536
    x, xs, w, ws, off = inputs(e, n, k, 90, seed=21, force_empty=force_empty)
    for g in force_empty:
        assert off[g] == off[g + 1]
    x = np.concatenate([x, np.zeros((10, k // 2), np.uint8)])
    xs = np.concatenate([xs, np.full((10, k // 32), 127, np.uint8)])
    ref = reference(x, xs, w, ws, off)
    assert np.isnan(ref[90:]).all()
    check(run(x, xs, w, ws, off, torch.float32, variant=V), ref, torch.float32, str(force_empty))


@pytest.mark.parametrize("per_expert", [1, 8, 24, 48, 96, 150])
def test_grouped_mid_is_the_librarys_choice_at_a_small_batch(per_expert):
    """8 experts of config 4's N and K, a few rows per expert: AUTO must give the bits of the kernel asked for by
    name, which is checked against the oracle (all rows up to 8 per expert, sampled rows beyond) and, element for
    element, against the table-driven tile kernels."""
    e, n, k = 8, 14336, 4096
    rows = e * per_expert
    x, xs, w, ws, off = inputs(e, n, k, rows, seed=3, lo=122, hi=132)
    c = run(x, xs, w, ws, off, torch.bfloat16, variant=V)
    assert np.array_equal(run(x, xs, w, ws, off, torch.bfloat16), c)
    for g in range(e):
        a, b = int(off[g]), int(off[g + 1])
        if b == a:
            continue
        pick = np.unique(np.concatenate([np.arange(a, b, max(1, (b - a) // 6)), [b - 1]]))
        ref = c_oracle.scaled_gemm_exact(x, w[g], xs, ws[g], rows=pick)
        assert_close(c[pick], ref, torch.bfloat16, f"expert {g}")
    tiles = run(x, xs, w, ws, off, torch.float32, variant=_lib.VARIANT_T128x128_W2x2)
    assert_close(c, tiles.astype(np.float64), torch.bfloat16, "all elements vs the tile kernel")


def test_grouped_mid_unsupported_cases_are_refused():
    e, n, k, rows = 4, 128, 512, 32           # fewer than four K tiles
    x, xs, w, ws, off = inputs(e, n, k, rows, seed=9)
    with pytest.raises((ValueError, RuntimeError)):
        run(x, xs, w, ws, off, torch.float32, variant=V)


@pytest.mark.parametrize("la", [RM, M32], ids=["a_scales_row_major", "a_scales_mfma32"])
@pytest.mark.parametrize("e,n,k,rows", [
    (8, 4096, 1024, 1280),    # 160 rows per expert: one pass of the 192-row block
    (8, 4096, 1024, 2048),    # 256: the 128x256 tiles would take two sparsely filled rounds, two passes here
    (8, 4096, 1024, 3072),    # 384: less than two rounds of 256x256 tiles, three passes here
    (16, 2048, 1024, 2900),   # 181 per expert
    (8, 4096, 1024, 4500),    # 563 per expert: back on the tile kernels (two well-filled rounds)
    (4, 4096, 1024, 1300),    # few experts of many rows: the tile kernels
])
def test_library_choice_beyond_160_rows_per_expert(e, n, k, rows, la):
    """Whichever kernel the library picks for a grouped problem of 160 .. 560 rows per expert (its estimate of the
    rounds either side would take; the groups of several 192-row passes among them), every group's rows against the
    exact oracle on the first, the last and 64 random columns, and bit-equal to the mid-M kernel asked for by name
    where that is what ran (same K order on every kernel: the two agree to the last bit anyway)."""
    x, xs, w, ws, off = inputs(e, n, k, rows, seed=e + rows, lo=120, hi=132)
    rng = np.random.default_rng(rows)
    cols = np.unique(np.concatenate([[0, 1, 127, 128, n - 1], rng.integers(0, n, 64)]))
    ref = reference(x, xs, w[:, cols], ws[:, cols], off)
    for dt in (torch.bfloat16, torch.float32):
        c = run(x, xs, w, ws, off, dt, lb=M32, la=la)
        assert not np.isnan(c).any(), "unwritten elements"
        check(c[:, cols], ref, dt, f"E={e} {rows}x{n}x{k} library's choice")
        by_name = run(x, xs, w, ws, off, dt, lb=M32, la=la, variant=V)
        assert np.array_equal(c, by_name)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("e,n,k,rows", [(8, 2880, 2880, 64), (4, 5760, 2880, 100), (6, 640, 1056, 333), (32, 256, 2848, 40)])
def test_grouped_mid_partial_last_k_tile(e, n, k, rows, dt):
    """K in whole scale groups but not in whole K tiles (2880: gpt-oss) with both scale tensors in MFMA32 order,
    whose zero padding cancels what the last K tile reads past the end of K (the next row, the next expert's first
    row, or nothing): by name and by the library's own choice, row-major and preshuffled expert weights; with
    row-major scales the kernel is refused by name and the library's choice runs the tile kernels."""
    x, xs, w, ws, off = inputs(e, n, k, rows, seed=e + rows + k)
    ref = reference(x, xs, w, ws, off)
    check(run(x, xs, w, ws, off, dt, lb=M32, la=M32, variant=V), ref, dt, f"E={e} {rows}x{n}x{k} by name")
    check(run(x, xs, w, ws, off, dt, lb=M32, la=M32), ref, dt, f"E={e} {rows}x{n}x{k} library's choice")
    if k % 64 == 0:
        check(run(x, xs, w, ws, off, dt, lb=M32, la=M32, pre=True, variant=V), ref, dt, f"E={e} {rows}x{n}x{k} preshuffled")
    check(run(x, xs, w, ws, off, dt), ref, dt, f"E={e} {rows}x{n}x{k} row-major scales")
    with pytest.raises((RuntimeError, ValueError)):
        run(x, xs, w, ws, off, dt, variant=V)
