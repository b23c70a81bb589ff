"""Torch-facing operators over the C ABI.  Torch supplies device memory and
the current stream; all arithmetic happens in the HIP library.

Calling convention kept from the reference launch path
(wave_lang/kernel/wave/compile.py:225-339, utils/run_utils.py:62-134):
tensors are passed positionally, non-contiguous inputs are silently made
contiguous, the output is pre-allocated by the caller and mutated in place,
the work is enqueued on the current stream without synchronising, and the
call returns None."""

from __future__ import annotations

import functools

import torch

from . import _lib

_OUT_DTYPES = {torch.float32: _lib.OUT_F32, torch.bfloat16: _lib.OUT_BF16}


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """``torch.cuda.device(d)`` only when ``d`` is not the current device already (the context manager costs
    several microseconds of host time per call, which shows on small problems)."""

    __slots__ = ("_ctx",)

    def __init__(self, device):
        idx = device.index if device.index is not None else torch.cuda.current_device()
        self._ctx = None if idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            self._ctx.__exit__(*exc)
        return False


def _as_u8(t: torch.Tensor, name: str) -> torch.Tensor:
    # the reference annotates these buffers i8 and its tests pass uint8
    if t.dtype not in (torch.uint8, torch.int8):
        raise ValueError(f"{name}: expected uint8/int8, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name}: expected a GPU tensor (there is no CPU path)")
    return t if t.is_contiguous() else t.contiguous()


def _check_out(out: torch.Tensor, shape) -> int:
    if out.dtype not in _OUT_DTYPES:
        raise ValueError(f"out: expected float32 or bfloat16, got {out.dtype}")
    if not out.is_cuda or not out.is_contiguous():
        raise ValueError("out: expected a contiguous GPU tensor")
    if tuple(out.shape) != tuple(shape):
        raise ValueError(f"out: expected shape {tuple(shape)}, got {tuple(out.shape)}")
    return _OUT_DTYPES[out.dtype]


def _scale_rows_ok(scale: torch.Tensor, rows: int, ks: int, layout: int, name: str) -> None:
    if layout == _lib.SCALE_ROW_MAJOR:
        if tuple(scale.shape) != (rows, ks):
            raise ValueError(f"{name}: expected shape {(rows, ks)}, got {tuple(scale.shape)}")
    elif layout == _lib.SCALE_PER_ROW:
        if tuple(scale.shape) != (rows,):
            raise ValueError(f"{name}: expected shape {(rows,)}, got {tuple(scale.shape)}")
    else:
        need = ((rows + 31) // 32 * 32) * ((ks + 7) // 8 * 8)
        if scale.numel() < need:
            raise ValueError(
                f"{name}: shuffled scales need {need} bytes (rows padded to 32, groups to 8), got {scale.numel()}")


@functools.lru_cache(maxsize=4096)
def workspace_bytes(m: int, n: int, k: int, split_k: int = 0, variant: int = _lib.VARIANT_AUTO) -> int:
    return int(_lib.load().wave_mxfp4_workspace_bytes(m, n, k, split_k, variant))


# One scratch buffer per (device, stream), grown on demand: the split-K partial
# sums and the re-laid-out scales of a call live there.  Calls on one stream are
# ordered, so they can share it; different streams get different buffers.
# A buffer that was handed out is never freed: a HIP graph captured while it was
# current keeps its address, so a buffer that a larger call supersedes moves to
# `_retired` and stays allocated until the process ends.  Buffers grow geometrically
# (the request rounded up to a power of two), so what a run of slowly growing problems
# leaves in `_retired` stays below the size of the live buffer.
_scratch: dict = {}
_retired: list = []
# signatures of mxfp4_gemm calls that passed every check: -> (m, n, k, out dtype code, a scale layout, scratch bytes)
_checked: dict = {}


def _grow_scratch(key, nbytes: int, alloc):
    """The cached buffer of `key` if it holds `nbytes`, else a new one from
    `alloc(nbytes)`; the superseded buffer is kept alive (see above)."""
    buf = _scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _retired.append(buf)
        buf = alloc(1 << max(int(nbytes) - 1, 0).bit_length())
        _scratch[key] = buf
    return buf


def _workspace(device, nbytes: int):
    if nbytes == 0:
        return None
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    return _grow_scratch(key, nbytes, lambda n: torch.empty(n, dtype=torch.uint8, device=device))


def mxfp4_gemm(x, x_scales, w_t, w_scales, out, *, a_scale_layout=_lib.SCALE_ROW_MAJOR,
               b_scale_layout=_lib.SCALE_ROW_MAJOR, b_layout=_lib.B_ROW_MAJOR, split_k=0,
               variant=_lib.VARIANT_AUTO, workspace=None) -> None:
    """``out[M, N] = dequant(x[M, K/2]) @ dequant(w_t[N, K/2]).T`` in place.
    Same arguments, in the same order, as the reference's compiled kernel
    (tests/kernel/wave_gemm_mxfp_test.py:194-201).  ``workspace`` is an optional
    uint8 GPU tensor of ``workspace_bytes(...)`` bytes; by default a buffer cached
    per device and stream is used, ``False`` runs without scratch.  ``split_k``: 0 lets the
    library split K where that pays (decode shapes with K > 8192, few-tile shapes with long K; the
    result is overwritten either way), 1 never splits, n > 1 splits n ways.

    Two more call shapes of the reference are taken as they are:
    * batched A with a shared B, ``x [B, M, K/2]``, ``x_scales [B, M, K/32]``,
      ``out [B, M, N]`` (tests/kernel/wave_gemm_mxfp_test.py:205-339): the batch
      is folded into the rows, which it is in memory;
    * one scale per row of A, ``x_scales [M]``, held for the whole row
      (wave_lang/kernel/wave/templates/test_kernels.py:75-135)."""
    lib = _lib.load()
    # A call whose shapes, types, device and options were checked before skips the checks (they cost more host
    # time than the launch of a small problem): contiguity is the one property a tensor of the same shape can lose.
    key = (x.shape, x_scales.shape, w_t.shape, w_scales.shape, out.shape, x.dtype, x_scales.dtype, w_t.dtype,
           w_scales.dtype, out.dtype, x.device, w_t.device, out.device, a_scale_layout, b_scale_layout, b_layout,
           split_k, variant)
    plan = _checked.get(key)
    if (plan is not None and workspace is None and x.is_contiguous() and x_scales.is_contiguous()
            and w_t.is_contiguous() and w_scales.is_contiguous() and out.is_contiguous()
            and x_scales.device == x.device and w_scales.device == x.device):
        m, n, k, od, asl, nbytes = plan
        device = x.device
        stream = torch.cuda.current_stream(device).cuda_stream
        ws_ptr = None
        if nbytes:
            buf = _scratch.get((device, stream))
            if buf is None or buf.numel() < nbytes:
                buf = _workspace(device, nbytes)
            ws_ptr = buf.data_ptr()
        with _on_device(device):
            st = lib.wave_mxfp4_gemm(x.data_ptr(), x_scales.data_ptr(), w_t.data_ptr(), w_scales.data_ptr(),
                                     out.data_ptr(), m, n, k, od, asl, b_scale_layout, b_layout, split_k, ws_ptr,
                                     nbytes if ws_ptr is not None else 0, variant, stream)
        _lib.check(st, "wave_mxfp4_gemm")
        return
    x = _as_u8(x, "x")
    w_t = _as_u8(w_t, "w_t")
    x_scales = _as_u8(x_scales, "x_scales")
    w_scales = _as_u8(w_scales, "w_scales")
    if x.dim() == 3:
        if a_scale_layout != _lib.SCALE_ROW_MAJOR:
            raise ValueError("batched x: scales must be row-major [B, M, K/32]")
        bsz, bm = x.shape[0], x.shape[1]
        if x_scales.dim() != 3 or tuple(x_scales.shape[:2]) != (bsz, bm):
            raise ValueError(f"x_scales: expected [{bsz}, {bm}, K/32], got {tuple(x_scales.shape)}")
        if out.dim() != 3 or tuple(out.shape[:2]) != (bsz, bm) or not out.is_contiguous():
            raise ValueError(f"out: expected a contiguous [{bsz}, {bm}, N], got {tuple(out.shape)}")
        x = x.reshape(bsz * bm, x.shape[2])
        x_scales = x_scales.reshape(bsz * bm, x_scales.shape[2])
        out = out.view(bsz * bm, out.shape[2])
    if x_scales.dim() == 1 and a_scale_layout == _lib.SCALE_ROW_MAJOR:
        a_scale_layout = _lib.SCALE_PER_ROW
    if x.dim() != 2 or w_t.dim() != 2:
        raise ValueError("x must be 2-D (or 3-D batched) and w_t 2-D")
    m, kp = x.shape
    n = w_t.shape[0]
    if w_t.shape[1] != kp:
        raise ValueError(f"x and w_t disagree on K/2: {kp} vs {w_t.shape[1]}")
    k = kp * 2
    if k % 32 != 0:
        raise ValueError(f"K = {k} must be a multiple of 32")
    ks = k // 32
    _scale_rows_ok(x_scales, m, ks, a_scale_layout, "x_scales")
    _scale_rows_ok(w_scales, n, ks, b_scale_layout, "w_scales")
    od = _check_out(out, (m, n))
    ws_ptr, ws_bytes = None, 0
    default_scratch = workspace is None
    if workspace is None:
        workspace = _workspace(x.device, workspace_bytes(m, n, k, split_k, variant))
    elif workspace is False:  # run without scratch: scales are read in the layout given
        workspace = None
    if workspace is not None:
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    if w_t.device != x.device or out.device != x.device or x_scales.device != x.device or w_scales.device != x.device:
        raise ValueError("all tensors must be on the same device")
    with _on_device(x.device):
        st = lib.wave_mxfp4_gemm(x.data_ptr(), x_scales.data_ptr(), w_t.data_ptr(), w_scales.data_ptr(),
                                 out.data_ptr(), m, n, k, od, a_scale_layout, b_scale_layout, b_layout,
                                 split_k, ws_ptr, ws_bytes, variant, _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp4_gemm")
    if default_scratch:  # remember the checked signature (as given by the caller: before any reshaping above)
        if len(_checked) > 4096:
            _checked.clear()
        _checked[key] = (m, n, k, od, a_scale_layout, workspace_bytes(m, n, k, split_k, variant))


def mxfp4_gemm_grouped(x, x_scales, w_t, w_scales, offsets, out, *, a_scale_layout=_lib.SCALE_ROW_MAJOR,
                       b_scale_layout=_lib.SCALE_ROW_MAJOR, b_layout=_lib.B_ROW_MAJOR,
                       variant=_lib.VARIANT_AUTO, workspace=None) -> None:
    """Grouped (MoE) GEMM: rows ``offsets[e]:offsets[e+1]`` of ``x`` times
    expert ``e``'s ``w_t[e]`` ``[N, K/2]``; ``offsets`` is an int32 GPU tensor
    of E+1 entries.  ``out`` is ``[rows, N]``; rows past ``offsets[-1]`` are
    left untouched.  ``workspace`` as in :func:`mxfp4_gemm`."""
    lib = _lib.load()
    x = _as_u8(x, "x")
    w_t = _as_u8(w_t, "w_t")
    x_scales = _as_u8(x_scales, "x_scales")
    w_scales = _as_u8(w_scales, "w_scales")
    if x.dim() != 2 or w_t.dim() != 3:
        raise ValueError("x must be [rows, K/2] and w_t [E, N, K/2]")
    if offsets.dtype != torch.int32 or not offsets.is_cuda or not offsets.is_contiguous():
        raise ValueError("offsets: expected a contiguous int32 GPU tensor")
    rows, kp = x.shape
    e, n, kp2 = w_t.shape
    if kp2 != kp:
        raise ValueError(f"x and w_t disagree on K/2: {kp} vs {kp2}")
    if offsets.numel() != e + 1:
        raise ValueError(f"offsets: expected {e + 1} entries, got {offsets.numel()}")
    k = kp * 2
    if k % 32 != 0:
        raise ValueError(f"K = {k} must be a multiple of 32")
    ks = k // 32
    _scale_rows_ok(x_scales, rows, ks, a_scale_layout, "x_scales")
    if b_scale_layout == _lib.SCALE_ROW_MAJOR:
        if tuple(w_scales.shape) != (e, n, ks):
            raise ValueError(f"w_scales: expected {(e, n, ks)}, got {tuple(w_scales.shape)}")
    else:
        need = e * ((n + 31) // 32 * 32) * ((ks + 7) // 8 * 8)
        if w_scales.numel() < need:
            raise ValueError(f"w_scales: shuffled scales need {need} bytes, got {w_scales.numel()}")
    od = _check_out(out, (rows, n))
    ws_ptr, ws_bytes = None, 0
    if workspace is None:
        workspace = _workspace(x.device, int(lib.wave_mxfp4_grouped_workspace_bytes(rows, n, k, e)))
    elif workspace is False:
        workspace = None
    if workspace is not None:
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    with _on_device(x.device):
        st = lib.wave_mxfp4_gemm_grouped(x.data_ptr(), x_scales.data_ptr(), w_t.data_ptr(),
                                         w_scales.data_ptr(), out.data_ptr(), offsets.data_ptr(), e, rows,
                                         n, k, od, a_scale_layout, b_scale_layout, b_layout, variant,
                                         ws_ptr, ws_bytes, _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp4_gemm_grouped")


def mxfp4_to_f32(x: torch.Tensor) -> torch.Tensor:
    """Packed e2m1 ``[R, K/2]`` -> f32 ``[R, K]``
    (wave_lang/kernel/wave/utils/mxfp_utils.py:60-83)."""
    lib = _lib.load()
    x = _as_u8(x, "x")
    rows, kp = x.shape
    out = torch.empty(rows, kp * 2, dtype=torch.float32, device=x.device)
    with _on_device(x.device):
        st = lib.wave_mxfp4_to_f32(x.data_ptr(), out.data_ptr(), rows, kp, _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp4_to_f32")
    return out


def e8m0_to_f32(s: torch.Tensor) -> torch.Tensor:
    """e8m0 bytes -> f32 ``2^(s-127)``, 255 -> NaN
    (wave_lang/kernel/wave/utils/mxfp_utils.py:86-95)."""
    lib = _lib.load()
    s = _as_u8(s, "s")
    out = torch.empty(s.shape, dtype=torch.float32, device=s.device)
    with _on_device(s.device):
        st = lib.wave_mxfp4_e8m0_to_f32(s.data_ptr(), out.data_ptr(), s.numel(), _stream_ptr(s.device))
    _lib.check(st, "wave_mxfp4_e8m0_to_f32")
    return out


def dequant(x: torch.Tensor, scales: torch.Tensor, scale_layout=_lib.SCALE_ROW_MAJOR) -> torch.Tensor:
    """``[R, K/2]`` codes and their scales -> f32 ``[R, K]`` (value times the
    scale of its 32-group), the operand the reference feeds to ``torch.mm``
    (wave_lang/kernel/wave/utils/mxfp_utils.py:135-143)."""
    lib = _lib.load()
    x = _as_u8(x, "x")
    scales = _as_u8(scales, "scales")
    rows, kp = x.shape
    k = kp * 2
    _scale_rows_ok(scales, rows, k // 32, scale_layout, "scales")
    out = torch.empty(rows, k, dtype=torch.float32, device=x.device)
    with _on_device(x.device):
        st = lib.wave_mxfp4_dequant(x.data_ptr(), scales.data_ptr(), out.data_ptr(), rows, k, scale_layout,
                                    _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp4_dequant")
    return out


def scale_convert(scale: torch.Tensor, rows: int, ks: int, src_layout: int, dst_layout: int) -> torch.Tensor:
    """Re-lays a scale tensor of the logical shape ``[rows, ks]`` out from one
    layout to another on the GPU.  Row-major results are ``[rows, ks]``; the
    others the padded ``[ceil(rows/32)*32, ceil(ks/8)*8]`` buffer."""
    lib = _lib.load()
    scale = _as_u8(scale, "scale")
    _scale_rows_ok(scale, rows, ks, src_layout, "scale")
    if dst_layout == _lib.SCALE_ROW_MAJOR:
        out = torch.empty(rows, ks, dtype=torch.uint8, device=scale.device)
    else:
        out = torch.empty((rows + 31) // 32 * 32, (ks + 7) // 8 * 8, dtype=torch.uint8, device=scale.device)
    with _on_device(scale.device):
        st = lib.wave_mxfp4_scale_convert(scale.data_ptr(), src_layout, out.data_ptr(), dst_layout, rows, ks,
                                          _stream_ptr(scale.device))
    _lib.check(st, "wave_mxfp4_scale_convert")
    return out


def e8m0_shuffle(scale: torch.Tensor) -> torch.Tensor:
    """Scale matrix ``[R, K/32]`` -> the tile order the kernels read with one
    dword per lane (wave_lang/kernel/wave/utils/mxfp_utils.py:113-128).

    Returns the PADDED buffer ``[ceil(R/32)*32, ceil(K/32/8)*8]``; when R is a
    multiple of 32 and K of 256 that is exactly the reference's result.  (The
    reference slices back to ``[R, K/32]``, which drops bytes of valid rows
    otherwise.)"""
    lib = _lib.load()
    scale = _as_u8(scale, "scale")
    rows, ks = scale.shape
    out = torch.empty((rows + 31) // 32 * 32, (ks + 7) // 8 * 8, dtype=torch.uint8, device=scale.device)
    with _on_device(scale.device):
        st = lib.wave_mxfp4_e8m0_shuffle(scale.data_ptr(), out.data_ptr(), rows, ks, _stream_ptr(scale.device))
    _lib.check(st, "wave_mxfp4_e8m0_shuffle")
    return out


def b_preshuffle(b: torch.Tensor) -> torch.Tensor:
    """``[N, K/2]`` packed weights -> same shape in the order a lane reads with
    one 16-byte load per MFMA operand
    (wave_lang/kernel/wave/utils/mxfp_utils.py:98-110)."""
    lib = _lib.load()
    b = _as_u8(b, "b")
    rows, kp = b.shape
    out = torch.empty_like(b)
    with _on_device(b.device):
        st = lib.wave_mxfp4_b_preshuffle(b.data_ptr(), out.data_ptr(), rows, kp, _stream_ptr(b.device))
    _lib.check(st, "wave_mxfp4_b_preshuffle")
    return out


_IN_DTYPES = {torch.float32: _lib.IN_F32, torch.bfloat16: _lib.IN_BF16, torch.float16: _lib.IN_F16}


def quantize_mxfp4(x: torch.Tensor, *, shuffle: bool = False, scale_layout: int | None = None):
    """``[R, K]`` f32 / bf16 / f16 -> ``(x_q [R, K/2] uint8, x_scales)``, the A
    (or B) operand pair of :func:`mxfp4_gemm`.  Same call shape as the quantiser
    the reference's benchmark uses, ``quant_func(x, shuffle=True)``
    (wave_lang/kernel/wave/perf/bench_mxfp4_comparison.py:1484-1486):
    ``shuffle=True`` writes the scales in ``e8m0_shuffle`` order.

    ``x_scales`` is ``[R, K/32]`` for the row-major layout, otherwise the padded
    buffer ``[ceil(R/32)*32, ceil(K/32/8)*8]`` in the tile order of
    ``scale_layout``."""
    lib = _lib.load()
    if x.dim() != 2:
        raise ValueError(f"x: expected [R, K], got shape {tuple(x.shape)}")
    if x.dtype not in _IN_DTYPES:
        raise ValueError(f"x: dtype {x.dtype} is not float32, bfloat16 or float16")
    if x.device.type != "cuda":
        raise ValueError("x: expected a device tensor")
    layout = scale_layout if scale_layout is not None else (_lib.SCALE_E8M0_SHUFFLE if shuffle else _lib.SCALE_ROW_MAJOR)
    x = x.contiguous()
    rows, k = x.shape
    if k % 32:
        raise ValueError(f"x: K = {k} is not a multiple of 32")
    ks = k // 32
    q = torch.empty(rows, k // 2, dtype=torch.uint8, device=x.device)
    if layout == _lib.SCALE_ROW_MAJOR:
        scales = torch.empty(rows, ks, dtype=torch.uint8, device=x.device)
    else:
        scales = torch.empty((rows + 31) // 32 * 32, (ks + 7) // 8 * 8, dtype=torch.uint8, device=x.device)
    with _on_device(x.device):
        st = lib.wave_mxfp4_quantize(x.data_ptr(), _IN_DTYPES[x.dtype], q.data_ptr(), scales.data_ptr(), rows, k,
                                     layout, _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp4_quantize")
    return q, scales


def _new_scales(rows: int, ks: int, layout: int, device) -> torch.Tensor:
    if layout == _lib.SCALE_ROW_MAJOR:
        return torch.empty(rows, ks, dtype=torch.uint8, device=device)
    return torch.empty((rows + 31) // 32 * 32, (ks + 7) // 8 * 8, dtype=torch.uint8, device=device)


def quantize_mxfp4_rows(x: torch.Tensor, row_ids: torch.Tensor, row_div: int = 1, *,
                        scale_layout: int = _lib.SCALE_ROW_MAJOR):
    """Quantise gathered rows: output row ``r`` is row ``row_ids[r] // row_div``
    of ``x [R, K]``; ids at or beyond ``R * row_div`` (the padding value of
    :func:`moe_align_block_size`) give zero rows.  With ``row_ids = sorted_ids``
    and ``row_div = top_k`` this is the per-expert gather of the repeated
    activations in the reference's MoE (tests/kernel/moe_test.py:113-127) fused
    into the quantiser.  Returns ``(q [len(row_ids), K/2], scales)``."""
    lib = _lib.load()
    if x.dim() != 2 or x.dtype not in _IN_DTYPES or x.device.type != "cuda":
        raise ValueError("x: expected a [R, K] float32 / bfloat16 / float16 device tensor")
    if row_ids.dtype != torch.int32 or row_ids.dim() != 1 or row_ids.device != x.device:
        raise ValueError("row_ids: expected a 1-D int32 tensor on x's device")
    x = x.contiguous()
    row_ids = row_ids.contiguous()
    src_rows, k = x.shape
    if k % 32:
        raise ValueError(f"x: K = {k} is not a multiple of 32")
    rows = row_ids.numel()
    q = torch.empty(rows, k // 2, dtype=torch.uint8, device=x.device)
    scales = _new_scales(rows, k // 32, scale_layout, x.device)
    with _on_device(x.device):
        st = lib.wave_mxfp4_quantize_rows(x.data_ptr(), _IN_DTYPES[x.dtype], src_rows, row_ids.data_ptr(), int(row_div),
                                          q.data_ptr(), scales.data_ptr(), rows, k, scale_layout,
                                          _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp4_quantize_rows")
    return q, scales


def moe_align_block_size(topk_ids: torch.Tensor, num_experts: int, block_size: int, sorted_ids: torch.Tensor,
                         expert_ids: torch.Tensor, num_tokens_post_pad: torch.Tensor,
                         expert_offsets: torch.Tensor | None = None) -> None:
    """Same arguments as the reference's ``moe_align_block_size_pytorch``
    (tests/kernel/moe/torch_kernels.py:10-92): all outputs are pre-allocated by
    the caller (int32) and filled in place.  ``expert_offsets`` (optional,
    ``num_experts + 1`` int32) receives the running sums of the padded counts."""
    lib = _lib.load()
    if topk_ids.dtype not in (torch.int32, torch.int64) or not topk_ids.is_cuda:
        raise ValueError("topk_ids: expected an int32 or int64 device tensor")
    for name, t in (("sorted_ids", sorted_ids), ("expert_ids", expert_ids),
                    ("num_tokens_post_pad", num_tokens_post_pad), ("expert_offsets", expert_offsets)):
        if t is not None and (t.dtype != torch.int32 or not t.is_contiguous() or t.device != topk_ids.device):
            raise ValueError(f"{name}: expected a contiguous int32 tensor on topk_ids' device")
    if expert_offsets is not None and expert_offsets.numel() < num_experts + 1:
        raise ValueError("expert_offsets: needs num_experts + 1 entries")
    if num_tokens_post_pad.numel() < 1:
        raise ValueError("num_tokens_post_pad: needs one entry")
    ids = topk_ids.contiguous()
    with _on_device(ids.device):
        st = lib.wave_mxfp4_moe_align_block_size(
            ids.data_ptr(), 1 if ids.dtype == torch.int64 else 0, ids.numel(), int(num_experts), int(block_size),
            sorted_ids.data_ptr(), sorted_ids.numel(), expert_ids.data_ptr(), expert_ids.numel(),
            num_tokens_post_pad.data_ptr(), expert_offsets.data_ptr() if expert_offsets is not None else None,
            _stream_ptr(ids.device))
    _lib.check(st, "wave_mxfp4_moe_align_block_size")


def _gated_args(gate: torch.Tensor, up: torch.Tensor):
    if gate.dim() != 2 or gate.shape != up.shape or gate.dtype != up.dtype or gate.device != up.device:
        raise ValueError("gate and up: expected two [M, N] tensors of one dtype on one device")
    if gate.dtype not in (torch.bfloat16, torch.float16) or not gate.is_cuda:
        raise ValueError(f"gate: expected a bfloat16 or float16 device tensor, got {gate.dtype}")
    # row strides are passed through (the halves of a [M, 2N] tensor are fine); anything else is copied
    gate = gate if gate.stride(1) == 1 else gate.contiguous()
    up = up if up.stride(1) == 1 else up.contiguous()
    return gate, up


def silu_and_mul(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``gate * up / (1 + exp(-gate))`` (tests/kernel/moe_test.py:39-40,69-79),
    f32 inside, rounded once to the inputs' dtype."""
    lib = _lib.load()
    gate, up = _gated_args(gate, up)
    rows, n = gate.shape
    if out is None:
        out = torch.empty(rows, n, dtype=gate.dtype, device=gate.device)
    elif out.shape != gate.shape or out.dtype != gate.dtype or out.stride(1) != 1:
        raise ValueError("out: expected the shape and dtype of gate, unit column stride")
    with _on_device(gate.device):
        st = lib.wave_mxfp4_silu_and_mul(gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.stride(0), up.stride(0),
                                         out.stride(0), _IN_DTYPES[gate.dtype], rows, n, _stream_ptr(gate.device))
    _lib.check(st, "wave_mxfp4_silu_and_mul")
    return out


def silu_and_mul_quantize(gate: torch.Tensor, up: torch.Tensor, *, scale_layout: int = _lib.SCALE_ROW_MAJOR):
    """:func:`silu_and_mul` followed by :func:`quantize_mxfp4` in one kernel
    (same bits, no ``[M, N]`` round trip): the A operand of the second expert
    GEMM.  Returns ``(q [M, N/2], scales)``."""
    lib = _lib.load()
    gate, up = _gated_args(gate, up)
    rows, n = gate.shape
    q = torch.empty(rows, n // 2, dtype=torch.uint8, device=gate.device)
    scales = _new_scales(rows, n // 32, scale_layout, gate.device)
    with _on_device(gate.device):
        st = lib.wave_mxfp4_silu_and_mul_quantize(gate.data_ptr(), up.data_ptr(), gate.stride(0), up.stride(0),
                                                  _IN_DTYPES[gate.dtype], q.data_ptr(), scales.data_ptr(), rows, n,
                                                  scale_layout, _stream_ptr(gate.device))
    _lib.check(st, "wave_mxfp4_silu_and_mul_quantize")
    return q, scales


def interleave_gate_up(t: torch.Tensor) -> torch.Tensor:
    """``[..., 2I, C]`` uint8 (gate rows, then up rows: packed weights or their row-major scales) -> the same shape
    with blocks of 32 rows alternating gate, up, ...: the weight order :func:`mxfp4_gemm_gated_quantize` takes."""
    lib = _lib.load()
    t = _as_u8(t, "t")
    if t.dim() < 2 or t.shape[-2] % 64 != 0:
        raise ValueError("expected [..., 2I, C] with I a multiple of 32")
    out = torch.empty_like(t)
    flat_in, flat_out = t.reshape(-1, t.shape[-2], t.shape[-1]), out.view(-1, t.shape[-2], t.shape[-1])
    with _on_device(t.device):
        for e in range(flat_in.shape[0]):
            st = lib.wave_mxfp4_interleave_gate_up(flat_in[e].data_ptr(), flat_out[e].data_ptr(), t.shape[-2] // 2,
                                                   t.shape[-1], _stream_ptr(t.device))
            _lib.check(st, "wave_mxfp4_interleave_gate_up")
    return out


def mxfp4_gemm_gated_quantize(x, x_scales, w_il, w_scales_il, offsets=None, *, a_scale_layout=_lib.SCALE_ROW_MAJOR,
                              b_scale_layout=_lib.SCALE_ROW_MAJOR, act_scale_layout=_lib.SCALE_MFMA32, workspace=None):
    """The first GEMM of a gated expert MLP with :func:`silu_and_mul_quantize` fused into its output: ``w_il``
    ``[E, 2I, K/2]`` (or ``[2I, K/2]`` with ``offsets=None``: dense) holds gate and up projections interleaved by
    :func:`interleave_gate_up`, as do its scales.  Returns ``(q [rows, I/2], scales)`` of ``silu(gate) * up``, the
    same bits as ``mxfp4_gemm_grouped`` (bf16 out) followed by ``silu_and_mul_quantize``.  Large batches run the
    persistent kernel, small grouped ones (the batches :func:`mxfp4_gemm_grouped` gives to the mid-M kernel: up to 160 rows per expert on
    average and some beyond) with ``b_scale_layout`` MFMA32 the
    mid-M kernel.  Raises ``ValueError`` (status "unsupported") where neither applies; the caller then runs the
    two calls."""
    lib = _lib.load()
    x, w_il = _as_u8(x, "x"), _as_u8(w_il, "w_il")
    x_scales, w_scales_il = _as_u8(x_scales, "x_scales"), _as_u8(w_scales_il, "w_scales_il")
    grouped = offsets is not None
    if x.dim() != 2 or w_il.dim() != (3 if grouped else 2):
        raise ValueError("x must be [rows, K/2] and w_il [E, 2I, K/2] (grouped) or [2I, K/2] (dense)")
    rows, kp = x.shape
    e = w_il.shape[0] if grouped else 0
    n = w_il.shape[-2]
    if w_il.shape[-1] != kp:
        raise ValueError(f"x and w_il disagree on K/2: {kp} vs {w_il.shape[-1]}")
    if n % 64 != 0:
        raise ValueError("w_il: 2I must be a multiple of 64")
    k, inter = kp * 2, n // 2
    if grouped and (offsets.dtype != torch.int32 or not offsets.is_cuda or offsets.numel() != e + 1):
        raise ValueError("offsets: expected a contiguous int32 GPU tensor of E + 1 entries")
    _scale_rows_ok(x_scales, rows, k // 32, a_scale_layout, "x_scales")
    q = torch.empty(rows, inter // 2, dtype=torch.uint8, device=x.device)
    scales = _new_scales(rows, inter // 32, act_scale_layout, x.device)
    if workspace is None:
        workspace = _workspace(x.device, int(lib.wave_mxfp4_grouped_workspace_bytes(rows, n, k, max(e, 1))))
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    with _on_device(x.device):
        st = lib.wave_mxfp4_gemm_gated_quantize(x.data_ptr(), x_scales.data_ptr(), w_il.data_ptr(), w_scales_il.data_ptr(),
                                                q.data_ptr(), scales.data_ptr(), offsets.data_ptr() if grouped else None,
                                                e, rows, n, k, a_scale_layout, b_scale_layout, act_scale_layout, ws_ptr,
                                                ws_bytes, _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp4_gemm_gated_quantize")
    return q, scales


_FP8_FORMATS = {torch.float8_e4m3fn: _lib.MXFP8_E4M3, torch.float8_e5m2: _lib.MXFP8_E5M2}


def mxfp8_b_preshuffle(b: torch.Tensor) -> torch.Tensor:
    """``[N, K]`` 8-bit weights (uint8 / int8 / float8) -> the same bytes in the order the B-direct MXFP8 kernel
    reads with one coalesced 16-byte load per lane (blocks of 32 rows x 128 bytes; the layout is this library's:
    the reference's ``b_preshuffle``, wave_lang/kernel/wave/utils/mxfp_utils.py:98-110, covers packed MXFP4 rows
    only).  N % 32 == 0, K % 128 == 0.  For :func:`mxfp8_gemm` with ``b_preshuffled=True``."""
    lib = _lib.load()
    dt = b.dtype
    if dt in _FP8_FORMATS or dt == torch.int8:
        b = b.view(torch.uint8)
    b = _as_u8(b, "b")
    if b.dim() != 2:
        raise ValueError("b must be [N, K]")
    rows, k = b.shape
    out = torch.empty_like(b)
    with _on_device(b.device):
        st = lib.wave_mxfp8_b_preshuffle(b.data_ptr(), out.data_ptr(), rows, k, _stream_ptr(b.device))
    _lib.check(st, "wave_mxfp8_b_preshuffle")
    return out.view(dt)


def mxfp8_gemm(x, x_scales, w_t, w_scales, out, *, elem_format=None,
               variant=_lib.VARIANT_AUTO, workspace=None, b_preshuffled=False,
               a_scale_layout=_lib.SCALE_ROW_MAJOR, b_scale_layout=_lib.SCALE_ROW_MAJOR) -> None:
    """``out[M, N] = (x * scales) @ (w_t * scales).T`` for MXFP8 operands:
    ``x [M, K]``, ``w_t [N, K]`` one byte per element, scales ``[R, K/32]`` e8m0
    (tests/kernel/wave_gemm_mxfp_test.py:416-501, which passes
    ``x.view(torch.int8)`` of ``float8_e5m2`` tensors).  float8 tensors carry
    their format; for uint8 / int8 views pass ``elem_format``, one value for both
    operands or a pair ``(x format, w_t format)`` (default e5m2, the
    reference's ``tkl.f8e5m2``).  With ``MXFP8_E2M1`` as one of the two formats that
    operand is ``[rows, K/2]`` packed MXFP4 against the 8-bit other (8-bit activations
    against 4-bit weights or the other way round, the mixed operands of
    wave_lang/kernel/wave/constraints.py:425-431; both 4-bit is :func:`mxfp4_gemm`).
    ``workspace`` as in :func:`mxfp4_gemm`.  ``b_preshuffled=True``: ``w_t`` comes from
    :func:`mxfp8_b_preshuffle` (a packed e2m1 ``w_t`` from :func:`b_preshuffle`) and the B-direct kernel
    runs (``x`` 8-bit, N % 256 == 0,
    K % 256 == 0, K >= 768; ``ValueError`` "unsupported" otherwise); only that call takes scale
    tensors in MFMA32 order (``a_scale_layout`` / ``b_scale_layout``)."""
    lib = _lib.load()
    given = tuple(elem_format) if isinstance(elem_format, (tuple, list)) else (elem_format, elem_format)
    if len(given) != 2:
        raise ValueError("elem_format is one format or a pair (x, w_t)")
    ops, fmts = [], []
    for name, t, fmt in (("x", x, given[0]), ("w_t", w_t, given[1])):
        if t.dtype in _FP8_FORMATS:
            if fmt is not None and fmt != _FP8_FORMATS[t.dtype]:
                raise ValueError(f"{name}: {t.dtype} does not match elem_format {fmt}")
            fmt = _FP8_FORMATS[t.dtype]
            t = t.view(torch.uint8)
        ops.append(_as_u8(t, name))
        fmts.append(_lib.MXFP8_E5M2 if fmt is None else fmt)
    x, w_t = ops
    x_scales = _as_u8(x_scales, "x_scales")
    w_scales = _as_u8(w_scales, "w_scales")
    x4, w4 = fmts[0] == _lib.MXFP8_E2M1, fmts[1] == _lib.MXFP8_E2M1
    if x4 and w4:
        raise ValueError("both operands e2m1: that is mxfp4_gemm")
    if x.dim() != 2 or w_t.dim() != 2:
        raise ValueError("x must be [M, K] and w_t [N, K] ([rows, K/2] for a packed e2m1 operand)")
    k = x.shape[1] * 2 if x4 else x.shape[1]
    if w_t.shape[1] != (k // 2 if w4 else k):
        raise ValueError("x must be [M, K] and w_t [N, K] ([rows, K/2] for a packed e2m1 operand)")
    m = x.shape[0]
    n = w_t.shape[0]
    if k % 128:
        raise ValueError(f"K = {k} must be a multiple of 128")
    if not b_preshuffled and (a_scale_layout != _lib.SCALE_ROW_MAJOR or b_scale_layout != _lib.SCALE_ROW_MAJOR):
        raise ValueError("scales in another order than row-major: only with b_preshuffled=True")
    _scale_rows_ok(x_scales, m, k // 32, a_scale_layout, "x_scales")
    _scale_rows_ok(w_scales, n, k // 32, b_scale_layout, "w_scales")
    od = _check_out(out, (m, n))
    ws_ptr, ws_bytes = None, 0
    if workspace is None:
        workspace = _workspace(x.device, int(lib.wave_mxfp8_workspace_bytes(m, n, k)))
    elif workspace is False:
        workspace = None
    if workspace is not None:
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    if b_preshuffled:
        with _on_device(x.device):
            st = lib.wave_mxfp8_gemm_b_preshuffled(x.data_ptr(), x_scales.data_ptr(), w_t.data_ptr(), w_scales.data_ptr(),
                                                   out.data_ptr(), m, n, k, fmts[0], fmts[1], od, a_scale_layout,
                                                   b_scale_layout, ws_ptr, ws_bytes, _stream_ptr(x.device))
        _lib.check(st, "wave_mxfp8_gemm_b_preshuffled")
        return
    with _on_device(x.device):
        st = lib.wave_mxfp8_gemm(x.data_ptr(), x_scales.data_ptr(), w_t.data_ptr(), w_scales.data_ptr(),
                                 out.data_ptr(), m, n, k, fmts[0], fmts[1], od, ws_ptr, ws_bytes, variant,
                                 _stream_ptr(x.device))
    _lib.check(st, "wave_mxfp8_gemm")
