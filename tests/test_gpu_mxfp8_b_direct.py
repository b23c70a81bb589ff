"""GPU: the MXFP8 GEMM with B in the library's preshuffled 8-bit order (wave_mxfp8_b_preshuffle,
wave_mxfp8_gemm_b_preshuffled): A through LDS, B straight into registers.  The layout against the numpy statement
of its definition (oracle/mxfp8_oracle.py, pinned byte by byte in tests/test_oracle_mxfp8.py); the GEMM against the oracle (oracle/mxfp8_oracle.py; bound as in test_gpu_mxfp8.py, the
reference's own test tests/kernel/wave_gemm_mxfp_test.py:416-501 uses atol 2e-3 / rtol 1e-3), bit for bit against
wave_mxfp8_gemm on the row-major operand (same products, same order of the K steps), and exactly on one-hot rows,
which read back single elements of dequantised B and so pin every position of the layout."""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import mxfp8_oracle as o8
from wave_amd import _lib

from gpu_util import DEV, to_gpu
from test_gpu_mxfp8 import assert_f32_close

pytestmark = pytest.mark.gpu
RM, M32 = _lib.SCALE_ROW_MAJOR, _lib.SCALE_MFMA32


def test_preshuffle_matches_its_definition():
    rng = np.random.default_rng(0)
    for n, k in [(32, 128), (64, 384), (256, 1024), (96, 2176)]:
        b = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
        got = wave_amd.mxfp8_b_preshuffle(torch.from_numpy(b).to(DEV)).cpu().numpy()
        assert np.array_equal(got, o8.b8_preshuffle(b)), (n, k)
    gb = torch.zeros(48, 128, dtype=torch.uint8, device=DEV)
    with pytest.raises(ValueError):
        wave_amd.mxfp8_b_preshuffle(gb)          # rows % 32
    with pytest.raises(ValueError):
        wave_amd.mxfp8_b_preshuffle(gb[:32, :64].contiguous())  # K % 128


def run(x, xs, w_t, ws, fmt, out_dtype=torch.float32, resident=False):
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    m, n, k = x.shape[0], w_t.shape[0], x.shape[1]
    b4 = isinstance(fmt, tuple) and fmt[1] == o8.E2M1
    wp = wave_amd.b_preshuffle(gw) if b4 else wave_amd.mxfp8_b_preshuffle(gw)
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    kw = {}
    if resident:
        gxs = wave_amd.scale_convert(gxs, m, k // 32, RM, M32)
        gws = wave_amd.scale_convert(gws, n, k // 32, RM, M32)
        kw = dict(a_scale_layout=M32, b_scale_layout=M32, workspace=False)
    wave_amd.mxfp8_gemm(gx, gxs, wp, gws, out, elem_format=fmt, b_preshuffled=True, **kw)
    torch.cuda.synchronize()
    return out


FMTS = {"e5m2": o8.E5M2, "e4m3": o8.E4M3, "e4m3_x_e5m2": (o8.E4M3, o8.E5M2), "e5m2_x_e4m3": (o8.E5M2, o8.E4M3),
        "e5m2_x_e2m1": (o8.E5M2, o8.E2M1), "e4m3_x_e2m1": (o8.E4M3, o8.E2M1)}


@pytest.mark.parametrize("fname", sorted(FMTS))
@pytest.mark.parametrize("m,n,k", [(256, 256, 768), (300, 512, 1024), (1, 256, 768), (513, 768, 1280)])
def test_against_oracle(m, n, k, fname):
    fmt = FMTS[fname]
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + n + k, fmt=fmt, scale_lo=120, scale_hi=134)
    ref = o8.scaled_gemm_mxfp8(x, w_t, xs, ws, fmt)
    c = run(x, xs, w_t, ws, fmt)
    assert_f32_close(c.cpu().numpy(), ref, f"{m}x{n}x{k} {fname}")
    again = run(x, xs, w_t, ws, fmt, resident=True)
    assert torch.equal(c, again), "scales handed over in MFMA32 order: other bits"


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fname", ["e5m2", "e4m3_x_e5m2", "e5m2_x_e2m1"])
@pytest.mark.parametrize("m,n,k", [(4352, 4096, 768), (4100, 4352, 1024), (2050, 8448, 1536)])
def test_more_tiles_than_cus_same_bits_as_the_row_major_call(m, n, k, fname, out_dtype):
    """272 / 289 / 297 tiles on 256 workgroups: every workgroup walks two output tiles, its request streams run
    across the tile boundary and the last tile row is ragged.  The row-major call runs the symmetric persistent
    kernel: the same MFMAs on the same operands in the same order."""
    fmt = FMTS[fname]
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=m + k, fmt=fmt, scale_lo=120, scale_hi=134)
    c = run(x, xs, w_t, ws, fmt, out_dtype=out_dtype)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    other = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    wave_amd.mxfp8_gemm(gx, gxs, gw, gws, other, elem_format=fmt)
    torch.cuda.synchronize()
    assert not bool(torch.isnan(c).any()), "unwritten elements"
    assert torch.equal(c, other)
    if out_dtype == torch.float32:
        rows = np.unique(np.concatenate([np.arange(0, m, 257), [m - 1, 255, 256]]))
        ref = o8.scaled_gemm_mxfp8(x[rows], w_t, xs[rows], ws, fmt)
        assert_f32_close(c.cpu().numpy()[rows], ref, f"{m}x{n}x{k}")


def test_one_hot_rows_read_back_every_position_of_b():
    """Row r of A is 1.0 at position (37 r) % K with scale 1: C[r, :] is column (37 r) % K of dequantised B,
    exactly.  4352 rows cover every K position of every 32-row block of B several times."""
    m, n, k = 4352, 4096, 768
    fmt = o8.E5M2
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=9, fmt=fmt, scale_lo=118, scale_hi=136)
    x[:] = 0
    xs[:] = 127
    one = int(np.nonzero(o8.E5M2_TABLE == 1.0)[0][0])
    pos = (np.arange(m) * 37) % k
    x[np.arange(m), pos] = one
    finite = np.isfinite(o8.E5M2_TABLE)
    w_t[~finite[w_t]] = one  # (no infinities or NaNs in B: 0 * inf would spread over the row)
    c = run(x, xs, w_t, ws, fmt).cpu().numpy()
    deq = o8.fp8_to_f64(w_t, fmt) * np.exp2(ws.astype(np.float64) - 127).repeat(32, axis=1)
    assert np.array_equal(c.astype(np.float64), deq[:, pos].T)


def test_one_hot_rows_read_back_every_position_of_a_4_bit_b():
    """The same through packed e2m1 weights in b_preshuffle order: every e2m1 value times a power of two is exact."""
    m, n, k = 4352, 4096, 768
    fmt = (o8.E4M3, o8.E2M1)
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=10, fmt=fmt, scale_lo=118, scale_hi=136)
    x[:] = 0
    xs[:] = 127
    one = int(np.nonzero(o8.E4M3_TABLE == 1.0)[0][0])
    pos = (np.arange(m) * 37) % k
    x[np.arange(m), pos] = one
    c = run(x, xs, w_t, ws, fmt).cpu().numpy()
    from oracle import mxfp4_oracle as o4
    b = o4.mxfp4_to_f32(w_t).astype(np.float64) * o4.e8m0_to_f32(ws).astype(np.float64).repeat(32, axis=1)
    assert np.array_equal(c, b[:, pos].T.astype(np.float32))


def test_what_the_kernel_does_not_serve_is_refused():
    m, n, k = 64, 256, 768
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=1, fmt=o8.E5M2)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    lib = _lib.load()
    nbytes = int(lib.wave_mxfp8_workspace_bytes(m, n, k))
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=DEV)

    def call(n_=n, k_=k, fa=_lib.MXFP8_E5M2, fb=_lib.MXFP8_E5M2, la=RM, lb=RM, ws_ptr=scratch.data_ptr(), ws_bytes=nbytes):
        return lib.wave_mxfp8_gemm_b_preshuffled(gx.data_ptr(), gxs.data_ptr(), gw.data_ptr(), gws.data_ptr(), out.data_ptr(),
                                                 m, n_, k_, fa, fb, 0, la, lb, ws_ptr, ws_bytes, None)

    assert call() == _lib.OK
    torch.cuda.synchronize()
    assert call(n_=128) == _lib.ERR_UNSUPPORTED            # whole 256-column tiles only
    assert call(k_=512) == _lib.ERR_UNSUPPORTED            # K >= 768
    assert call(k_=640) == _lib.ERR_UNSUPPORTED            # pairs of K tiles
    assert call(fa=_lib.MXFP8_E2M1) == _lib.ERR_UNSUPPORTED
    assert call(la=_lib.SCALE_E8M0_SHUFFLE) == _lib.ERR_UNSUPPORTED
    assert call(ws_ptr=None, ws_bytes=0) == _lib.ERR_UNSUPPORTED   # row-major scales need the scratch
    assert call(fa=3) == _lib.ERR_BAD_ENUM
    assert call(n_=100) == _lib.ERR_BAD_SHAPE


def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    names = sorted(FMTS)
    return [(i, int(rng.integers(1, 1400)), 256 * int(rng.integers(1, 9)), 256 * int(rng.integers(3, 11)),
             names[int(rng.integers(0, len(names)))], bool(rng.integers(0, 2)), bool(rng.integers(0, 2)))
            for i in range(count)]


@pytest.mark.parametrize("case", _random_cases(16, seed=31), ids=lambda c: f"{c[0]}-{c[1]}x{c[2]}x{c[3]}-{c[4]}")
def test_random_shapes_same_bits_as_the_row_major_call_and_close_to_the_oracle(case):
    """Seeded shapes nobody picked by hand (1 .. 6 x 8 tiles, K = 768 .. 2560): the row-major call runs the tile
    kernel or the symmetric persistent one, all with the K steps in the same order."""
    i, m, n, k, fname, bf16, resident = case
    fmt = FMTS[fname]
    out_dtype = torch.bfloat16 if bf16 else torch.float32
    x, xs, w_t, ws = o8.make_inputs_mxfp8(m, n, k, seed=500 + i, fmt=fmt, scale_lo=118, scale_hi=136)
    c = run(x, xs, w_t, ws, fmt, out_dtype=out_dtype, resident=resident)
    gx, gxs, gw, gws = to_gpu(x, xs, w_t, ws)
    other = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    # (without scratch: with it the library cuts the K of the few-tile cases into parts, which are summed apart)
    wave_amd.mxfp8_gemm(gx, gxs, gw, gws, other, elem_format=fmt, workspace=False)
    torch.cuda.synchronize()
    assert torch.equal(c, other), case
    if not bf16:
        rows = np.unique(np.r_[0:min(m, 3), m // 2, m - 1])
        ref = o8.scaled_gemm_mxfp8(x[rows], w_t, xs[rows], ws, fmt)
        assert_f32_close(c.cpu().numpy()[rows], ref, str(case))


def test_a_beyond_2_gib():
    """A of 2.15 GB (262444 rows of 8192 bytes): the descriptors are based at each tile, so rows on either side of
    the 2 GiB byte boundary (row 262144), the first and last tiles and rows at random must come out right; the
    symmetric kernel on the row-major B gives every element a second opinion."""
    m, n, k = 262144 + 300, 256, 8192
    fmt = o8.E4M3
    g = torch.Generator(device=DEV).manual_seed(77)
    x = torch.randint(0, 256, (m, k), dtype=torch.uint8, device=DEV, generator=g)
    x = torch.where((x & 0x7F) == 0x7F, x - 1, x)   # (no NaN codes)
    w = torch.randint(0, 256, (n, k), dtype=torch.uint8, device=DEV, generator=g)
    w = torch.where((w & 0x7F) == 0x7F, w - 1, w)
    xs = torch.randint(122, 132, (m, k // 32), dtype=torch.uint8, device=DEV, generator=g)
    ws = torch.randint(122, 132, (n, k // 32), dtype=torch.uint8, device=DEV, generator=g)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp8_gemm(x, xs, wave_amd.mxfp8_b_preshuffle(w), ws, out, elem_format=fmt, b_preshuffled=True)
    other = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp8_gemm(x, xs, w, ws, other, elem_format=fmt)
    torch.cuda.synchronize()
    assert torch.equal(out, other)
    rng = np.random.default_rng(5)
    rows = np.unique(np.concatenate([[0, 1, 255, 256, 262143, 262144, 262145, m - 2, m - 1], rng.integers(0, m, 24)]))
    idx = torch.from_numpy(rows).to(DEV)
    ref = o8.scaled_gemm_mxfp8(x[idx].cpu().numpy(), w.cpu().numpy(), xs[idx].cpu().numpy(), ws.cpu().numpy(), fmt)
    got = out[idx].float().cpu().numpy()
    tol = 2.0 ** -7 * np.abs(ref) + 1e-4 * np.abs(ref).max()
    assert (np.abs(got - ref) <= tol).all(), "beyond one bf16 ulp + 1e-4 * max"
