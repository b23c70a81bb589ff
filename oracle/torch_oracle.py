"""CPU port of the reference's torch path, op for op, used as the timed CPU
baseline and as a third statement of the GEMM.  TEST INFRASTRUCTURE ONLY.

Follows wave_lang/kernel/wave/utils/mxfp_utils.py:60-95,131-143: expand each
byte to two nibbles, gather a 16-entry table, broadcast ``2^(s-127)`` over
each 32-group, multiply elementwise, then one f32 ``torch.mm``."""

from __future__ import annotations

import time

import torch

SCALE_GROUP_SIZE = 32

_LUT = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
        -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def mxfp4_to_f32(x: torch.Tensor) -> torch.Tensor:
    """(wave_lang/kernel/wave/utils/mxfp_utils.py:60-83)"""
    x = x.repeat_interleave(2, dim=1)
    x[:, ::2] = x[:, ::2] & 0xF
    x[:, 1::2] = x[:, 1::2] >> 4
    return torch.tensor(_LUT, dtype=torch.float32, device=x.device)[x.long()]


def e8m0_to_f32(x: torch.Tensor) -> torch.Tensor:
    """(wave_lang/kernel/wave/utils/mxfp_utils.py:86-95); takes the bytes
    already widened to f32 like the reference's caller does."""
    nan_mask = x == 255
    out = 2 ** ((x - 127).to(torch.float32))
    out[nan_mask] = float("nan")
    return out


def torch_scaled_gemm_mxfp4(x, w_t, x_scales, w_scales, timings=None):
    """``C = deq(x) @ deq(w_t).T`` with ``w_t`` stored [N, K/2]
    (wave_lang/kernel/wave/utils/mxfp_utils.py:131-143).  ``timings``, when a
    dict, receives the dequantise and matmul wall times in seconds."""
    t0 = time.perf_counter()
    x_f32 = mxfp4_to_f32(x)
    w_f32 = mxfp4_to_f32(w_t)
    xs = e8m0_to_f32(x_scales.repeat_interleave(SCALE_GROUP_SIZE, dim=1).to(torch.float32))
    ws = e8m0_to_f32(w_scales.repeat_interleave(SCALE_GROUP_SIZE, dim=1).to(torch.float32))
    a = x_f32 * xs
    b = w_f32 * ws
    t1 = time.perf_counter()
    out = torch.mm(a, b.T)
    t2 = time.perf_counter()
    if timings is not None:
        timings["dequant_s"] = t1 - t0
        timings["matmul_s"] = t2 - t1
    return out
