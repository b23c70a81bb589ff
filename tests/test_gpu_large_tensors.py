"""GPU: operands and results beyond 2 GiB / 4 GiB, the sizes at which a 32-bit byte offset wraps.

The reference's own largest MXFP4 cases are batched 16384^3 problems (tests/kernel/wave_gemm_mxfp_test.py:296,344:
A of 1 GiB and more, C in f32 up to 8 GiB).  Here every kernel addresses an operand through buffer descriptors
based at its own tile (64-bit pointer arithmetic) with 32-bit offsets inside the tile; these cases put a tile on
either side of every 2 GiB / 4 GiB byte boundary of A, B and C:

  (a) C beyond 4 GiB:  M = 131072 (8 x 16384 rows folded), N = 16384, f32 out; K = 512 (one tile per workgroup)
      and K = 1024 (persistent kernel)
  (b) A beyond 2 GiB:  M = 131372, K = 32768, N = 256 (persistent kernel, last round cut along K)
  (c) B beyond 2 GiB:  M = 16 and 32, N = 2^20, K = 8192 on the decode kernels (B = 4 GiB)

Inputs are drawn on the device.  Rows (for (c): columns) around every boundary, in the first and last tiles and at
random are gathered on the device and compared with the exact oracle; (a) and (b) also check the checksum
identities C . 1 = deq(A) . (deq(B)^T . 1) and 1^T . C = (1^T . deq(A)) . deq(B)^T over EVERY row and column, so a
tile written to the wrong place, or not at all, shows wherever it is.
"""

import numpy as np
import pytest
import torch

import wave_amd
from oracle import c_oracle
from wave_amd import _lib

from gpu_util import DEV, assert_close

pytestmark = pytest.mark.gpu


def device_inputs(m, n, k, seed, lo=124, hi=130):
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, device=DEV, generator=g)
    w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=DEV, generator=g)
    xs = torch.randint(lo, hi + 1, (m, k // 32), dtype=torch.uint8, device=DEV, generator=g)
    ws = torch.randint(lo, hi + 1, (n, k // 32), dtype=torch.uint8, device=DEV, generator=g)
    return x, xs, w, ws


def rows_around(m, boundaries, seed, extra=8):
    rng = np.random.default_rng(seed)
    rows = {0, 1, 31, 32, 255, 256, m - 257, m - 256, m - 2, m - 1}
    for b in boundaries:
        rows.update(range(b - 2, b + 3))
        rows.update((b - 256, b + 255))
    rows.update(int(r) for r in rng.integers(0, m, extra))
    return np.array(sorted(r for r in rows if 0 <= r < m), dtype=np.int64)


def check_rows(out, x, xs, w, ws, rows, dt, what):
    idx = torch.from_numpy(rows).to(DEV)
    got = out[idx].float().cpu().numpy()
    ref = c_oracle.scaled_gemm_exact(x[idx].cpu().numpy(), w.cpu().numpy(), xs[idx].cpu().numpy(), ws.cpu().numpy())
    assert_close(got, ref, dt, what)


def check_sums(out, x, xs, w, ws, rel):
    """Row and column sums of all of C against the dequantised operands (f64 on the device, chunked)."""
    a = wave_amd.dequant(x, xs).double()
    b = wave_amd.dequant(w, ws).double()
    row_ref = a @ b.sum(dim=0)
    col_ref = a.sum(dim=0) @ b.t()
    m = out.shape[0]
    row_sum = torch.empty(m, dtype=torch.float64, device=DEV)
    row_abs = torch.empty(m, dtype=torch.float64, device=DEV)
    col_sum = torch.zeros(out.shape[1], dtype=torch.float64, device=DEV)
    col_abs = torch.zeros(out.shape[1], dtype=torch.float64, device=DEV)
    for r0 in range(0, m, 8192):
        c = out[r0:r0 + 8192].double()
        assert not torch.isnan(c).any(), f"rows {r0}..: unwritten or NaN elements"
        row_sum[r0:r0 + 8192] = c.sum(dim=1)
        row_abs[r0:r0 + 8192] = c.abs().sum(dim=1)
        col_sum += c.sum(dim=0)
        col_abs += c.abs().sum(dim=0)
    assert bool(((row_sum - row_ref).abs() <= rel * row_abs + 1e-9 * row_ref.abs().max()).all()), "row sums"
    assert bool(((col_sum - col_ref).abs() <= rel * col_abs + 1e-9 * col_ref.abs().max()).all()), "column sums"


@pytest.mark.parametrize("k", [512, 1024])
def test_c_beyond_4_gib_f32(k):
    m, n = 131072, 16384                      # C = 8 GiB in f32: row 65536 starts at byte 2^32
    x, xs, w, ws = device_inputs(m, n, k, seed=k)
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    assert out.numel() * 4 > 1 << 32
    # the reference's shape of the case: a batch of 8 x [16384, K/2] activations against one B
    wave_amd.mxfp4_gemm(x.view(8, m // 8, k // 2), xs.view(8, m // 8, k // 32), w, ws, out.view(8, m // 8, n))
    torch.cuda.synchronize()
    check_rows(out, x, xs, w, ws, rows_around(m, [32768, 65536, 98304], seed=k), torch.float32, f"C > 4 GiB, K = {k}")
    check_sums(out, x, xs, w, ws, rel=1e-4)


def test_a_beyond_2_gib_bf16():
    m, n, k = 131372, 256, 32768              # A = 2.15 GB: row 131072 starts at byte 2^31
    x, xs, w, ws = device_inputs(m, n, k, seed=7)
    assert x.numel() > 1 << 31
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    wave_amd.mxfp4_gemm(x, xs, w, ws, out)
    torch.cuda.synchronize()
    check_rows(out, x, xs, w, ws, rows_around(m, [65536, 131072], seed=3), torch.bfloat16, "A > 2 GiB")
    check_sums(out, x, xs, w, ws, rel=2.0 ** -7)   # bf16: at most half an ulp (2^-8) per element, and slack


@pytest.mark.parametrize("m,variant", [(16, _lib.VARIANT_AUTO), (1, _lib.VARIANT_AUTO), (32, _lib.VARIANT_AUTO),
                                       (32, _lib.VARIANT_MID_M)])
def test_b_beyond_2_gib_decode_kernels(m, variant):
    n, k = 1 << 20, 8192                      # B = 4 GiB: row 2^19 starts at byte 2^31
    x, xs, w, ws = device_inputs(m, n, k, seed=m, lo=120, hi=134)
    assert w.numel() == 1 << 32
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    try:
        wave_amd.mxfp4_gemm(x, xs, w, ws, out, variant=variant)
    except RuntimeError as e:
        # a kernel named by the caller may refuse a shape it cannot address; the library's own choice may not
        assert variant != _lib.VARIANT_AUTO and "unsupported" in str(e), e
        return
    torch.cuda.synchronize()
    assert not bool(torch.isnan(out.float()).any())
    cols = rows_around(n, [1 << 18, 1 << 19, 3 << 18], seed=m, extra=40)
    idx = torch.from_numpy(cols).to(DEV)
    got = out[:, idx].float().cpu().numpy()
    ref = c_oracle.scaled_gemm_exact(x.cpu().numpy(), w[idx].cpu().numpy(), xs.cpu().numpy(), ws[idx].cpu().numpy())
    assert_close(got, ref, torch.bfloat16, f"B > 2 GiB, M = {m}")
    # every column: the column sums against deq(A)'s column sums times deq(B)^T, chunk by chunk of B
    asum = wave_amd.dequant(x, xs).double().sum(dim=0)
    for n0 in range(0, n, 1 << 16):
        b = wave_amd.dequant(w[n0:n0 + (1 << 16)], ws[n0:n0 + (1 << 16)]).double()
        c = out[:, n0:n0 + (1 << 16)].double()
        ref_sum = b @ asum
        assert bool(((c.sum(dim=0) - ref_sum).abs() <= 2.0 ** -7 * c.abs().sum(dim=0) + 1e-5 * ref_sum.abs().max()).all()), n0  # (the second term: f32 summation noise of an element near zero)
