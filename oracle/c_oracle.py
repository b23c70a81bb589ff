"""ctypes binding of the plain-C oracle (``mxfp4_oracle.c``).  TEST
INFRASTRUCTURE ONLY: imported by the tests, the smoke check and the
CPU-baseline leg of the benchmark, never by the product package."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmxfp4_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (seconds)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmxfp4_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_SO)
        i64, p = ctypes.c_int64, ctypes.c_void_p
        _lib.orc_mxfp4_to_f32.argtypes = [p, i64, i64, p]
        _lib.orc_e8m0_to_f32.argtypes = [p, i64, p]
        _lib.orc_dequant_f32.argtypes = [p, p, i64, i64, p]
        _lib.orc_gemm_f32.argtypes = [p, p, p, p, p, i64, i64, i64]
        _lib.orc_gemm_f32.restype = ctypes.c_int
        _lib.orc_gemm_exact.argtypes = [p, p, p, p, p, i64, i64, i64, p, i64]
        _lib.orc_gemm_exact.restype = ctypes.c_int
        _lib.orc_e8m0_shuffle_index.argtypes = [i64, i64, i64]
        _lib.orc_e8m0_shuffle_index.restype = i64
        _lib.orc_e8m0_shuffle_padded.argtypes = [p, i64, i64, p]
        _lib.orc_b_preshuffle_index.argtypes = [i64, i64, i64]
        _lib.orc_b_preshuffle_index.restype = i64
        _lib.orc_b_preshuffle.argtypes = [p, i64, i64, p]
    return _lib


def _u8(a):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    return a, a.ctypes.data


def mxfp4_to_f32(q):
    q, qp = _u8(q)
    out = np.empty((q.shape[0], q.shape[1] * 2), dtype=np.float32)
    lib().orc_mxfp4_to_f32(qp, q.shape[0], q.shape[1], out.ctypes.data)
    return out


def e8m0_to_f32(s):
    s, sp = _u8(s)
    out = np.empty(s.shape, dtype=np.float32)
    lib().orc_e8m0_to_f32(sp, s.size, out.ctypes.data)
    return out


def dequant_f32(q, scale):
    q, qp = _u8(q)
    scale, sp = _u8(scale)
    k = q.shape[1] * 2
    out = np.empty((q.shape[0], k), dtype=np.float32)
    lib().orc_dequant_f32(qp, sp, q.shape[0], k, out.ctypes.data)
    return out


def scaled_gemm_f32(x, w_t, x_scales, w_scales):
    x, xp = _u8(x)
    w_t, wp = _u8(w_t)
    xs, xsp = _u8(x_scales)
    ws, wsp = _u8(w_scales)
    m, n, k = x.shape[0], w_t.shape[0], x.shape[1] * 2
    out = np.empty((m, n), dtype=np.float32)
    rc = lib().orc_gemm_f32(xp, xsp, wp, wsp, out.ctypes.data, m, n, k)
    if rc:
        raise MemoryError("orc_gemm_f32")
    return out


def scaled_gemm_exact(x, w_t, x_scales, w_scales, rows=None):
    x, xp = _u8(x)
    w_t, wp = _u8(w_t)
    xs, xsp = _u8(x_scales)
    ws, wsp = _u8(w_scales)
    m, n, k = x.shape[0], w_t.shape[0], x.shape[1] * 2
    if rows is None:
        nr, rp = m, None
    else:
        rows = np.ascontiguousarray(rows, dtype=np.int64)
        nr, rp = rows.size, rows.ctypes.data
    out = np.empty((nr, n), dtype=np.float64)
    rc = lib().orc_gemm_exact(xp, xsp, wp, wsp, out.ctypes.data, m, n, k, rp, nr)
    if rc:
        raise MemoryError("orc_gemm_exact")
    return out


def e8m0_shuffle_padded(scale):
    scale, sp = _u8(scale)
    m, ks = scale.shape
    sm, sn = (m + 255) // 256 * 256, (ks + 7) // 8 * 8
    out = np.empty((sm, sn), dtype=np.uint8)
    lib().orc_e8m0_shuffle_padded(sp, m, ks, out.ctypes.data)
    return out


def b_preshuffle(b):
    b, bp = _u8(b)
    out = np.empty_like(b)
    lib().orc_b_preshuffle(bp, b.shape[0], b.shape[1], out.ctypes.data)
    return out
