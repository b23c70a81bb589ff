"""Host-side MXFP4 helpers with the reference's names
(wave_lang/kernel/wave/utils/mxfp_utils.py): the seeded input generator and
the two layout shuffles.  The element decoders run in the HIP library.  The
reference's ``torchScaledGemmMXFP4`` (its numerical oracle) is not part of
this package; the test-suite carries its own restatement."""

from __future__ import annotations

import torch

from .... import mxfp4 as _ops

SCALE_GROUP_SIZE = 32


def generate_gemm_afp4wfp4_inputs(shape, device=None, seed: int = 5, scale_range=(124, 128)):
    """Random packed MXFP4 inputs and e8m0 scales, same shapes, seed, draw
    order and ranges as wave_lang/kernel/wave/utils/mxfp_utils.py:20-57.
    Returns ``(x [M,K/2], w [K/2,N] (a transposed view), x_scales [M,K/32],
    w_scales [N,K/32])``; kernels take ``w.T.contiguous()``."""
    if device is None:
        device = torch.device("cuda" if torch.cuda.is_available() else "cpu")
    m, n, k = shape
    torch.manual_seed(seed)
    x_low = torch.randint(0, 16, (m, k // 2), dtype=torch.uint8, device=device)
    x_high = torch.randint(0, 16, (m, k // 2), dtype=torch.uint8, device=device)
    x = x_low | (x_high << 4)
    w_low = torch.randint(0, 16, (n, k // 2), dtype=torch.uint8, device=device)
    w_high = torch.randint(0, 16, (n, k // 2), dtype=torch.uint8, device=device)
    w = (w_low | (w_high << 4)).T
    lo, hi = scale_range
    x_scales = torch.randint(lo, hi, (k // SCALE_GROUP_SIZE, m), dtype=torch.uint8, device=device)
    w_scales = torch.randint(lo, hi, (k // SCALE_GROUP_SIZE, n), dtype=torch.uint8, device=device)
    return x, w, x_scales.T.contiguous(), w_scales.T.contiguous()


def mxfp4_to_f32(x: torch.Tensor) -> torch.Tensor:
    """(mxfp_utils.py:60-83) on the GPU."""
    return _ops.mxfp4_to_f32(x)


def e8m0_to_f32(x: torch.Tensor) -> torch.Tensor:
    """(mxfp_utils.py:86-95) on the GPU; takes the scale bytes."""
    return _ops.e8m0_to_f32(x)


def b_preshuffle(b: torch.Tensor) -> torch.Tensor:
    """(mxfp_utils.py:98-110).  GPU tensors go through the HIP kernel; CPU
    tensors (offline weight preparation) through the same reshape/permute."""
    if b.is_cuda:
        return _ops.b_preshuffle(b)
    n, kp = b.shape
    return b.view(n // 16, 16, kp // 32, 2, 16).permute(0, 2, 3, 1, 4).contiguous().view(n, kp)


def e8m0_shuffle(scale: torch.Tensor) -> torch.Tensor:
    """(mxfp_utils.py:113-128).  Returns the buffer padded to 32 rows and 8
    groups (identical to the reference's result whenever that one is
    lossless, i.e. rows % 32 == 0 and groups % 8 == 0)."""
    if scale.is_cuda:
        return _ops.e8m0_shuffle(scale)
    m, n = scale.shape
    sm, sn = (m + 31) // 32 * 32, (n + 7) // 8 * 8
    padded = torch.zeros(sm, sn, dtype=scale.dtype)
    padded[:m, :n] = scale
    padded = padded.view(sm // 32, 2, 16, sn // 8, 2, 4).permute(0, 3, 5, 2, 4, 1).contiguous()
    return padded.view(sm, sn)
