"""GPU parity at the five benchmark configurations, full size.

First line: the exact oracle on rows of EVERY 256-row M tile (at least 8 per
tile, all residues mod 32; about 500 rows at 8192^3, which the OpenMP C oracle
does in seconds).  Second line: every element against the independent
one-thread-per-element device kernel (itself pinned against the oracle on the
same rows), and size-independent identities (checksum of checksums)."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from oracle import mxfp4_oracle as orc
from wave_amd import _lib

from gpu_util import F32_TIGHT as F32_TIGHT_
from gpu_util import (BF16_ABS, BF16_REL, DEV, TILE_VARIANTS, assert_bf16_close, assert_close,
                      assert_f32_close, run_gemm, to_gpu)

pytestmark = pytest.mark.gpu


def sample_rows(m, per_tile, seed, tile=256, lo=0):
    """Rows of [lo, lo + m) for the exact oracle: in EVERY `tile`-row M tile (counted from `lo`, where a
    group's tiles start) one row per 32-row block, at residue (4 * block + tile index) % 32, so that four
    consecutive tiles cover every residue mod 32 (the MFMA's row-in-tile, lane and scale-block positions),
    plus `per_tile - 8` random rows of the tile, plus the corners of the first and last tiles."""
    rng = np.random.default_rng(seed)
    rows = {r for r in (0, 1, 31, 32, tile - 1, tile, m // 2, m - tile, m - 2, m - 1) if 0 <= r < m}
    for t in range((m + tile - 1) // tile):
        base, height = t * tile, min(tile, m - t * tile)
        for b in range((height + 31) // 32):
            r = base + 32 * b + (4 * b + t) % 32
            rows.add(min(r, m - 1))
        for r in rng.integers(0, height, size=max(per_tile - 8, 0)):
            rows.add(base + int(r))
    return np.array(sorted(rows), dtype=np.int64) + lo


def checksum_identities(c, x, xs, w_t, ws, rel_per_elem):
    """C . 1 == deq(A) . (deq(B)^T . 1) and 1^T . C == (1^T . deq(A)) . deq(B)^T,
    each within the sum of the per-element rounding allowances."""
    c = c.astype(np.float64)
    a = orc.dequant_f32(x, xs).astype(np.float64)
    b = orc.dequant_f32(w_t, ws).astype(np.float64)
    row_sum = a @ b.sum(axis=0)
    col_sum = a.sum(axis=0) @ b.T
    allow_r = rel_per_elem * np.abs(c).sum(axis=1) + 1e-6 * np.abs(row_sum).max()
    allow_c = rel_per_elem * np.abs(c).sum(axis=0) + 1e-6 * np.abs(col_sum).max()
    assert np.all(np.abs(c.sum(axis=1) - row_sum) <= allow_r)
    assert np.all(np.abs(c.sum(axis=0) - col_sum) <= allow_c)


def test_config1_1024_cubed_f32_seed0():
    m = n = k = 1024
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=0, scale_lo=124, scale_hi=130)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    for vname, v in dict(TILE_VARIANTS, auto=_lib.VARIANT_AUTO, naive=_lib.VARIANT_NAIVE).items():
        assert_f32_close(run_gemm(x, xs, w_t, ws, torch.float32, variant=v), ref, vname)
    # the reference's own f32 path agrees with the exact oracle at this size
    assert_f32_close(orc.scaled_gemm_f32(x, w_t, xs, ws), ref, "f32 oracle")


def test_config2_8192_cubed_bf16_seed1():
    m = n = k = 8192
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=1, scale_lo=124, scale_hi=130)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    rows = sample_rows(m, 16, seed=1)      # about 500 rows, at least 8 in each of the 32 M tiles
    assert len(rows) >= 8 * 32 and set(rows % 32) == set(range(32))
    assert all(((rows >= t * 256) & (rows < (t + 1) * 256)).sum() >= 8 for t in range(32))
    ref_rows = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)

    naive = torch.empty(m, n, dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gw, gws, naive, variant=_lib.VARIANT_NAIVE)
    naive = naive.cpu().numpy()
    assert_f32_close(naive[rows], ref_rows, "naive kernel vs oracle rows")

    for vname in ("auto", "t256x256_w2x2", "t256x256_w4x2"):
        v = dict(TILE_VARIANTS, auto=_lib.VARIANT_AUTO)[vname]
        out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, variant=v)
        c = out.float().cpu().numpy()
        assert_bf16_close(c[rows], ref_rows, f"{vname} vs oracle rows")
        assert_bf16_close(c, naive, f"{vname} vs naive kernel, all elements")
    checksum_identities(c, x, xs, w_t, ws, rel_per_elem=BF16_REL / 2 + BF16_ABS)


@pytest.mark.parametrize("m", [1, 16, 32])
def test_config3_decode_shapes_bf16_seed2(m):
    n, k = 28672, 8192
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=2, scale_lo=120, scale_hi=134)
    ref = c_oracle.scaled_gemm_exact(x, w_t, xs, ws)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)

    def run(**kw):
        out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        wave_amd.mxfp4_gemm(gx, gxs, gw, gws, out, **kw)
        return out.float().cpu().numpy()

    assert_bf16_close(run(), ref, "auto (skinny)")
    for splits in (2, 4, 8):
        assert_bf16_close(run(split_k=splits), ref, f"skinny split {splits}")
        assert_bf16_close(run(split_k=splits, variant=_lib.VARIANT_T128x128_W2x2), ref, f"tile split {splits}")
    # preshuffled weights and shuffled weight scales (static, prepared once)
    gwp = wave_amd.b_preshuffle(gw)
    gwss = wave_amd.e8m0_shuffle(gws)
    out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp4_gemm(gx, gxs, gwp, gwss, out, b_layout=_lib.B_PRESHUFFLE,
                        b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert_bf16_close(out.float().cpu().numpy(), ref, "preshuffled B + shuffled B scales")


def grouped_inputs(e, n, k, rows, seed, force_empty=()):
    off = orc.make_group_offsets(e, rows, seed, force_empty=force_empty)
    x, xs, _, _ = orc.make_inputs(rows, 1, k, seed, scale_lo=124, scale_hi=130)
    rng = np.random.default_rng(seed + 100)
    w = rng.integers(0, 256, size=(e, n, k // 2), dtype=np.uint8)
    ws = rng.integers(124, 131, size=(e, n, k // 32), dtype=np.uint8)
    return x, xs, w, ws, off


def run_grouped(x, xs, w, ws, off, out_dtype, **kw):
    gx, gxs, gw, gws, goff = to_gpu(x, xs, w, ws, off)
    out = torch.full((x.shape[0], w.shape[1]), float("nan"), dtype=out_dtype, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out, **kw)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def test_config4_grouped_moe_bf16_seed3():
    e, n, k, rows = 8, 14336, 4096, 8192
    x, xs, w, ws, off = grouped_inputs(e, n, k, rows, seed=3)
    assert off[-1] == rows and len(set(np.diff(off))) > 1          # ragged
    # rows of every expert against the exact per-expert oracle: at least 8 in every 256-row tile of the
    # expert's range (tiles start at the expert's first row), all residues mod 32 per expert
    picks, ref = [], []
    for g in range(e):
        lo, hi = int(off[g]), int(off[g + 1])
        if hi == lo:
            continue
        rows_g = sample_rows(hi - lo, 12, seed=30 + g, lo=lo)
        assert rows_g.min() >= lo and rows_g.max() < hi
        if hi - lo >= 1024:
            assert set((rows_g - lo) % 32) == set(range(32))
        ref.append(c_oracle.scaled_gemm_exact(x, w[g], xs, ws[g], rows=rows_g))
        picks.append(rows_g)
    picks, ref = np.concatenate(picks), np.concatenate(ref)
    naive = run_grouped(x, xs, w, ws, off, torch.float32, variant=_lib.VARIANT_NAIVE)
    assert_f32_close(naive[picks], ref, "naive grouped vs oracle rows")
    for vname in ("auto", "t256x256_w2x2", "t128x128_w2x2"):
        v = dict(TILE_VARIANTS, auto=_lib.VARIANT_AUTO)[vname]
        c = run_grouped(x, xs, w, ws, off, torch.bfloat16, variant=v)
        assert_bf16_close(c[picks], ref, f"{vname} vs oracle rows")
        assert_bf16_close(c, naive, f"{vname} vs naive kernel, all elements")


@pytest.mark.parametrize("force_empty", [(0,), (3, 4), (7,), (0, 1, 2, 3, 4, 5, 6)])
def test_grouped_empty_groups_and_small(force_empty):
    e, n, k, rows = 8, 160, 512, 700
    x, xs, w, ws, off = grouped_inputs(e, n, k, rows, seed=21, force_empty=force_empty)
    for g in force_empty:
        assert off[g] == off[g + 1]
    ref = orc.scaled_gemm_grouped_exact(x, xs, w, ws, off)
    for v in (_lib.VARIANT_AUTO, _lib.VARIANT_T256x256_W4x2, _lib.VARIANT_NAIVE):
        c = run_grouped(x, xs, w, ws, off, torch.float32, variant=v)
        assert_f32_close(c, ref, str(v))
        # without the scratch buffer the scales are read as given instead of re-laid out first: same bits
        assert np.array_equal(run_grouped(x, xs, w, ws, off, torch.float32, variant=v, workspace=False), c)


def test_grouped_rows_past_last_offset_untouched_and_layouts():
    e, n, k, rows = 4, 96, 256, 300
    x, xs, w, ws, off = grouped_inputs(e, n, k, 260, seed=22)
    x = np.concatenate([x, np.zeros((40, k // 2), np.uint8)])
    xs = np.concatenate([xs, np.full((40, k // 32), 127, np.uint8)])
    ref = orc.scaled_gemm_grouped_exact(x, xs, w, ws, off)
    c = run_grouped(x, xs, w, ws, off, torch.float32)
    assert_f32_close(c[:260], ref[:260])
    assert np.isnan(c[260:]).all()                                  # never written
    # preshuffled expert weights and shuffled expert scales
    wp = np.stack([orc.b_preshuffle(w[g]) for g in range(e)])
    wss = np.stack([orc.e8m0_shuffle_padded(ws[g])[:96] for g in range(e)])
    c2 = run_grouped(x, xs, wp, wss, off, torch.float32, b_layout=_lib.B_PRESHUFFLE,
                     b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert np.array_equal(c2[:260], c[:260])


def test_config5_edge_shape_shuffled_scales_f32_seed4():
    m, n, k = 4093, 6144, 7168
    x, xs, w_t, ws = orc.make_inputs(m, n, k, seed=4, scale_lo=100, scale_hi=154)
    rows = sample_rows(m, 16, seed=4)      # at least 8 rows in each of the 16 M tiles (the last one 253 rows)
    assert all(((rows >= t * 256) & (rows < (t + 1) * 256)).sum() >= 8 for t in range(16))
    ref_rows = c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)

    def run(a_s, b_s, **kw):
        out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
        wave_amd.mxfp4_gemm(gx, a_s, gw, b_s, out, **kw)
        return out.cpu().numpy()

    plain = run(gxs, gws)
    assert_f32_close(plain[rows], ref_rows, "row-major scales vs oracle rows")
    naive = run(gxs, gws, variant=_lib.VARIANT_NAIVE)
    assert_f32_close(naive[rows], ref_rows, "naive kernel vs oracle rows")
    assert_f32_close(plain, naive, "row-major scales vs naive kernel, all elements")

    # scales in the preshuffled tile order: B clean (6144 % 32 == 0), A padded to 4096 rows
    xs_sh = wave_amd.e8m0_shuffle(gxs)
    ws_sh = wave_amd.e8m0_shuffle(gws)
    assert xs_sh.shape == (4096, 224) and ws_sh.shape == (6144, 224)
    assert np.array_equal(xs_sh.cpu().numpy(), orc.e8m0_shuffle_padded(xs)[:4096])
    shuffled = run(xs_sh, ws_sh, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE)
    assert np.array_equal(shuffled, plain)                          # same arithmetic, same bits
    direct = run(xs_sh, ws_sh, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                 workspace=False)
    # read in place, no pre-pass.  (With scratch the library may cut the tiles of a sparsely filled last round
    # along K, which changes the order of the sums: compared within f32 accumulation noise, not bit for bit.)
    assert_f32_close(direct, plain, "no scratch vs scratch")
    assert np.array_equal(run(gxs, gws, workspace=False), direct)
    # and with preshuffled B on top
    gwp = wave_amd.b_preshuffle(gw)
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm(gx, xs_sh, gwp, ws_sh, out, a_scale_layout=_lib.SCALE_E8M0_SHUFFLE,
                        b_scale_layout=_lib.SCALE_E8M0_SHUFFLE, b_layout=_lib.B_PRESHUFFLE)
    assert np.array_equal(out.cpu().numpy(), plain)
    checksum_identities(plain, x, xs, w_t, ws, rel_per_elem=2e-6)


def test_grouped_many_expert_rows_with_scratch():
    """E * N beyond 65535 blocks of 32 scale rows (E = 128, N = 16416: 2.1 M rows of B scales, 269 MB of B at
    K = 256): the scale re-layout in front of the grouped GEMM must serve it, with and without the workspace."""
    e, n, k, rows = 128, 16416, 256, 200
    assert e * n > 65535 * 32
    off = orc.make_group_offsets(e, rows, seed=40)
    x, xs, _, _ = orc.make_inputs(rows, 1, k, 40, scale_lo=124, scale_hi=130)
    gen = torch.Generator(device=DEV).manual_seed(40)
    gw = torch.randint(0, 256, (e, n, k // 2), dtype=torch.uint8, device=DEV, generator=gen)
    gws = torch.randint(124, 131, (e, n, k // 32), dtype=torch.uint8, device=DEV, generator=gen)
    gx, gxs, goff = to_gpu(x, xs, off)
    out = torch.full((rows, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out)
    c = out.cpu().numpy()
    out.fill_(float("nan"))
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out, workspace=False)
    assert np.array_equal(out.cpu().numpy(), c)
    for g in sorted(set(np.searchsorted(off, np.arange(rows), side="right") - 1))[::9]:   # some of the used experts
        lo, hi = int(off[g]), int(off[g + 1])
        ref = c_oracle.scaled_gemm_exact(x[lo:hi], gw[g].cpu().numpy(), xs[lo:hi], gws[g].cpu().numpy())
        assert_f32_close(c[lo:hi], ref, f"expert {g}")


@pytest.mark.parametrize("la,lb", [("rm", "rm"), ("m32", "rm"), ("rm", "m32"), ("m32", "m32")])
def test_grouped_persistent_path_scale_layouts_and_ragged_starts(la, lb):
    """The table-driven persistent kernel (more 256x256 tiles than CUs) with each scale tensor row-major or already
    in MFMA32 order: groups start at rows that are no multiples of 32, so a tile's lanes find their scales in two
    neighbouring blocks of A's scale tensor; a NaN scale in a group's last row must poison that row only (the rows
    of the next group that share its tile's padding are not written by it).  Rows of every tile against the oracle."""
    e, n, k, rows = 5, 4096, 1024, 4700
    x, xs, w, ws, off = grouped_inputs(e, n, k, rows, seed=77)
    assert any(int(o) % 32 for o in off[1:-1])
    last = int(off[2]) - 1                      # last row of group 1
    xs[last, 5] = 255
    gx, gxs, gw, gws, goff = to_gpu(x, xs, w, ws, off)
    m32 = _lib.SCALE_MFMA32
    if la == "m32":
        gxs = wave_amd.scale_convert(gxs, rows, k // 32, _lib.SCALE_ROW_MAJOR, m32)
    if lb == "m32":
        gws = torch.stack([wave_amd.scale_convert(gws[g], n, k // 32, _lib.SCALE_ROW_MAJOR, m32) for g in range(e)])
    out = torch.full((rows + 3, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out[:rows], variant=_lib.VARIANT_T256x256_W4x2,
                                a_scale_layout=m32 if la == "m32" else _lib.SCALE_ROW_MAJOR,
                                b_scale_layout=m32 if lb == "m32" else _lib.SCALE_ROW_MAJOR)
    torch.cuda.synchronize()
    c = out.cpu().numpy()
    assert np.isnan(c[rows:]).all() and np.isnan(c[last]).all()
    assert not np.isnan(np.delete(c[:rows], last, 0)).any()
    for g in range(e):
        lo, hi = int(off[g]), int(off[g + 1])
        pick = np.unique(np.concatenate([np.arange(lo, hi, 37), np.arange(max(lo, hi - 3), hi)]))
        pick = pick[pick != last]
        ref = c_oracle.scaled_gemm_exact(x, w[g], xs, ws[g], rows=pick)
        assert_f32_close(c[pick], ref, f"expert {g} {la}/{lb}")


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("e,n,k,rows", [(4, 2048, 14336, 9300), (8, 4096, 2048, 4200), (3, 1024, 8192, 16600)])
def test_grouped_persistent_path_sparse_last_round_cut_along_k(e, n, k, rows, dt):
    """A few rounds of tiles of which the last gives less than half of the workgroups one (296-320 tiles of 256x256
    on 256 CUs and the like): its tiles are cut along K over the idle workgroups, the f32 parts summed by a second
    launch; whether and how is decided on the device, where the tile count is known (56 and 32 K tiles: 3 and 8
    parts; 8 K tiles: too short to pay, the tiles stay whole).  Rows of every tile against the oracle, every element against the one-tile-per-workgroup kernel, rows past the last offset untouched."""
    x, xs, w, ws, off = grouped_inputs(e, n, k, rows, seed=e * 5 + 1)
    tiles = int(sum((int(off[g + 1]) - int(off[g]) + 255) // 256 for g in range(e))) * (n // 256)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert tiles > cus and 0 < tiles % cus <= cus // 2, "the case is meant to leave a sparse last round"
    gx, gxs, gw, gws, goff = to_gpu(x, xs, w, ws, off)
    out = torch.full((rows + 2, n), float("nan"), dtype=dt, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out[:rows], variant=_lib.VARIANT_T256x256_W4x2)
    torch.cuda.synchronize()
    c = out.float().cpu().numpy()
    assert np.isnan(c[rows:]).all() and not np.isnan(c[:rows]).any()
    for g in range(e):
        lo, hi = int(off[g]), int(off[g + 1])
        pick = np.unique(np.concatenate([np.arange(lo, hi, 97), np.arange(lo, hi, 256), np.arange(lo + 255, hi, 256), [hi - 1]]))
        ref = c_oracle.scaled_gemm_exact(x, w[g], xs, ws[g], rows=pick)
        assert_close(c[pick], ref, dt, f"expert {g}")
    other = torch.full((rows, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, other, variant=_lib.VARIANT_T128x128_W2x2, workspace=False)
    torch.cuda.synchronize()
    o = other.cpu().numpy()
    assert np.abs(c[:rows] - o).max() <= (4e-6 if dt == torch.float32 else 2.0 ** -7) * np.abs(o).max()


def torch_seeded_inputs(m, n, k, seed, scale_lo, scale_hi):
    """The configuration's operands drawn the way the reference draws its own (torch.manual_seed(seed), then the
    draw order of wave_lang/kernel/wave/utils/mxfp_utils.py:37-57 through the host mirror's generator), on the CPU
    so that the bytes do not depend on the GPU's random number generator."""
    from wave_amd.kernel.wave.utils.mxfp_utils import generate_gemm_afp4wfp4_inputs

    x, w, xs, ws = generate_gemm_afp4wfp4_inputs((m, n, k), device="cpu", seed=seed, scale_range=(scale_lo, scale_hi + 1))
    return x.numpy(), xs.numpy(), w.T.contiguous().numpy(), ws.numpy()


@pytest.mark.parametrize("name,m,n,k,dt,seed,lo,hi", [
    ("cfg1", 1024, 1024, 1024, torch.float32, 0, 124, 130),
    ("cfg2", 8192, 8192, 8192, torch.bfloat16, 1, 124, 130),
    ("cfg3_m16", 16, 28672, 8192, torch.bfloat16, 2, 120, 134),
    ("cfg3_m128", 128, 28672, 8192, torch.bfloat16, 2, 120, 134),
    ("cfg5", 4093, 6144, 7168, torch.float32, 4, 100, 154),
])
def test_configs_with_torch_seeded_inputs(name, m, n, k, dt, seed, lo, hi):
    """The same configurations on inputs seeded with torch.manual_seed(n) (the other tests of this file draw them
    with numpy's generator): the library's own kernel choice against the exact oracle, whole C for the small ones,
    at least 8 rows of every 256-row M tile for the large ones."""
    x, xs, w_t, ws = torch_seeded_inputs(m, n, k, seed, lo, hi)
    assert x.shape == (m, k // 2) and w_t.shape == (n, k // 2) and xs.min() >= lo and xs.max() <= hi
    c = run_gemm(x, xs, w_t, ws, dt)
    if m * n <= 1 << 22:
        assert_close(c, c_oracle.scaled_gemm_exact(x, w_t, xs, ws), dt, name)
    else:
        rows = sample_rows(m, 8, seed=seed)
        assert_close(c[rows], c_oracle.scaled_gemm_exact(x, w_t, xs, ws, rows=rows), dt, name)


def test_grouped_persistent_path_survives_malformed_offsets():
    """Offsets that are not non-decreasing ([0, T, 0, T, ...]: every other group is the whole tensor, 40 tiles of
    256 rows against a table capacity of 18) are clamped, not validated: the table's last band is cut to the tiles
    that were written, so the walk reads no unwritten entry (wave_amd/csrc/mxfp4_group_table.h, checked on the CPU
    by tests/test_group_table_host.py).  The call must return, and every 256-column block of every row of C holds
    either nothing (a dropped tile) or that row's product with one of the experts that own it."""
    e, n, k, T = 8, 4096, 1024, 2560
    x, xs, w, ws, _ = grouped_inputs(e, n, k, T, seed=91)
    off = np.array([0, T] * 4 + [0], dtype=np.int32)
    gx, gxs, gw, gws, goff = to_gpu(x, xs, w, ws, off)
    out = torch.full((T, n), float("nan"), dtype=torch.float32, device=DEV)
    wave_amd.mxfp4_gemm_grouped(gx, gxs, gw, gws, goff, out, variant=_lib.VARIANT_T256x256_W4x2)
    torch.cuda.synchronize()
    c = out.cpu().numpy()
    pick = np.unique(np.concatenate([np.arange(0, T, 61), np.arange(255, T, 256)]))
    refs = [c_oracle.scaled_gemm_exact(x, w[g], xs, ws[g], rows=pick) for g in (0, 2, 4, 6)]
    # (tiles of different experts that cover the same rows are written concurrently: an element is one expert's or
    # another's, and which may differ from element to element)
    got = c[pick]
    dropped = np.isnan(got)
    err = np.min([np.abs(np.where(dropped, ref, got) - ref) for ref in refs], axis=0)
    assert err.max() <= F32_TIGHT_ * max(np.abs(ref).max() for ref in refs)
    blocks = dropped.reshape(len(pick), n // 256, 256)
    assert (blocks.all(axis=2) | ~blocks.any(axis=2)).all(), "a dropped tile is dropped whole"
    assert not dropped.all()
