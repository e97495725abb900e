"""Tensor-level entry points over the C ABI (one function per kernel).

These take and return ``torch`` tensors on an AMD GPU and do nothing but
validate, allocate outputs and pass raw pointers to ``libdaisy_hip.so``.
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from . import _lib

ATTN_SCALE = 0.12  # the reference's constant softmax scale (models/daisy/attention.py:88)


def _check_bf16(name: str, t: torch.Tensor, ndim: int) -> None:
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
    if t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")
    if t.stride(-1) != 1:
        raise ValueError(f"{name} must be contiguous in its last dim")


def prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *,
                      window: Optional[int], scale: float = ATTN_SCALE,
                      cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                      doc_start: Optional[torch.Tensor] = None,
                      out: Optional[torch.Tensor] = None, k_out: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Sliding-window causal attention over ``[B, T, H, D]`` bf16 tensors.

    ``cos``/``sin`` (fp32 ``[>=T, D/2]``) rotate q and k inside the call;
    ``doc_start`` (int32 ``[T]``) confines each query to its document; ``window``
    counts the visible keys including the query itself (``None``/``<=0`` = full
    causal).  Returns ``(o, k_rot)``: ``o`` is ``[B, T, H, D]`` bf16 and ``k_rot``
    the rotated keys (``None`` without ``cos``/``sin``).

    Contract of ``doc_start``: ``0 <= doc_start[t] <= t`` and non-decreasing in ``t`` (the kernel
    picks the key tiles of a block of queries from the block's first row).  It is not checked
    here, since that would synchronise; ``check_doc_start`` does, for callers that want it.
    """
    dev = _lib.require_gpu(q, k, v, cos, sin, doc_start, out, k_out)
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_bf16(name, t, 4)
    B, T, H, D = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"q, k, v shapes differ: {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    if (cos is None) != (sin is None):
        raise ValueError("cos and sin must be given together")
    if cos is not None:
        for name, t in (("cos", cos), ("sin", sin)):
            if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != D // 2 or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous fp32 [rows, {D // 2}] table, got {tuple(t.shape)} {t.dtype}")
            torch._assert(T <= t.shape[0], f"Rotary buffers too small {t.shape[0]} < {T}")
    if doc_start is not None:
        if doc_start.dtype != torch.int32 or doc_start.shape != (T,) or not doc_start.is_contiguous():
            raise ValueError("doc_start must be a contiguous int32 [T] tensor")
    if out is None:
        out = torch.empty((B, T, H, D), dtype=torch.bfloat16, device=dev)
    else:
        _check_bf16("out", out, 4)
    if cos is not None and k_out is None:
        k_out = torch.empty((B, T, H, D), dtype=torch.bfloat16, device=dev)
    if k_out is not None:
        _check_bf16("k_out", k_out, 4)
        if cos is None:
            raise ValueError("k_out is only produced when cos/sin are given")
    w = 0 if window is None else int(window)
    flags = 0
    lib = _lib.load()
    with _lib.on_device(dev):
        rc = lib.daisy_prefill_fwd(
            q.data_ptr(), _lib.strides(q, (0, 1, 2)),
            k.data_ptr(), _lib.strides(k, (0, 1, 2)),
            v.data_ptr(), _lib.strides(v, (0, 1, 2)),
            _lib.ptr(cos), _lib.ptr(sin), _lib.ptr(doc_start),
            out.data_ptr(), _lib.strides(out, (0, 1, 2)),
            _lib.ptr(k_out), None if k_out is None else _lib.strides(k_out, (0, 1, 2)),
            B, T, H, D, w, float(scale), flags, _lib.current_stream(dev))
    _lib.check(rc, "daisy_prefill_fwd")
    return out, k_out


def _check_f32(name: str, t: torch.Tensor, ndim: int) -> None:
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    if t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")
    if t.stride(-1) != 1:
        raise ValueError(f"{name} must be contiguous in its last dim")


def prefill_attention_f32(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *,
                          window: Optional[int], scale: float = ATTN_SCALE,
                          cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                          doc_start: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``prefill_attention`` on fp32 ``[B, T, H, D]`` tensors with fp32 arithmetic (``daisy_prefill_fwd_f32``):
    the mode of a module with fp32 parameters.  Any even ``D <= 256``.  Returns fp32 ``(o, k_rot)``."""
    dev = _lib.require_gpu(q, k, v, cos, sin, doc_start)
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_f32(name, t, 4)
    B, T, H, D = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"q, k, v shapes differ: {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    if (cos is None) != (sin is None):
        raise ValueError("cos and sin must be given together")
    if cos is not None:
        for name, t in (("cos", cos), ("sin", sin)):
            if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != D // 2 or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous fp32 [rows, {D // 2}] table, got {tuple(t.shape)} {t.dtype}")
            torch._assert(T <= t.shape[0], f"Rotary buffers too small {t.shape[0]} < {T}")
    if doc_start is not None:
        if doc_start.dtype != torch.int32 or doc_start.shape != (T,) or not doc_start.is_contiguous():
            raise ValueError("doc_start must be a contiguous int32 [T] tensor")
    out = torch.empty((B, T, H, D), dtype=torch.float32, device=dev)
    k_out = torch.empty((B, T, H, D), dtype=torch.float32, device=dev) if cos is not None else None
    d3 = (0, 1, 2)
    lib = _lib.load()
    with _lib.on_device(dev):
        rc = lib.daisy_prefill_fwd_f32(
            q.data_ptr(), _lib.strides(q, d3), k.data_ptr(), _lib.strides(k, d3), v.data_ptr(), _lib.strides(v, d3),
            _lib.ptr(cos), _lib.ptr(sin), _lib.ptr(doc_start),
            out.data_ptr(), _lib.strides(out, d3),
            _lib.ptr(k_out), None if k_out is None else _lib.strides(k_out, d3),
            B, T, H, D, 0 if window is None else int(window), float(scale), _lib.current_stream(dev))
    _lib.check(rc, "daisy_prefill_fwd_f32")
    return out, k_out


def decode_attention_f32(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                         k_rows: Optional[torch.Tensor], v_rows: Optional[torch.Tensor], *,
                         n_rows: int, new_idx: int, scale: float = ATTN_SCALE,
                         cos_row: Optional[torch.Tensor] = None, sin_row: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``decode_attention`` on fp32 tensors with fp32 arithmetic (``daisy_decode_fwd_f32``); the
    cache rows ``[B, H, rows, D]`` are only read."""
    dev = _lib.require_gpu(q, k_new, v_new, k_rows, v_rows, cos_row, sin_row)
    for name, t in (("q", q), ("k_new", k_new), ("v_new", v_new)):
        _check_f32(name, t, 3)
    B, H, D = q.shape
    if k_new.shape != q.shape or v_new.shape != q.shape:
        raise ValueError("q, k_new, v_new must all be [B, H, D]")
    if k_rows is not None:
        _check_f32("k_rows", k_rows, 4)
        _check_f32("v_rows", v_rows, 4)
    out = torch.empty((B, H, D), dtype=torch.float32, device=dev)
    lib = _lib.load()
    with _lib.on_device(dev):
        rc = lib.daisy_decode_fwd_f32(
            q.data_ptr(), _lib.strides(q, (0, 1)), k_new.data_ptr(), _lib.strides(k_new, (0, 1)),
            v_new.data_ptr(), _lib.strides(v_new, (0, 1)),
            _lib.ptr(k_rows), None if k_rows is None else _lib.strides(k_rows, (0, 1, 2)),
            _lib.ptr(v_rows), None if v_rows is None else _lib.strides(v_rows, (0, 1, 2)),
            _lib.ptr(cos_row), _lib.ptr(sin_row), out.data_ptr(), _lib.strides(out, (0, 1)),
            B, H, D, int(n_rows), int(new_idx), 0, float(scale), _lib.current_stream(dev))
    _lib.check(rc, "daisy_decode_fwd_f32")
    return out


def check_doc_start(doc_start: torch.Tensor) -> None:
    """Raises ``ValueError`` unless ``0 <= doc_start[t] <= t`` and ``doc_start`` does not decrease
    (the contract of ``prefill_attention``).  Synchronises with the device."""
    pos = torch.arange(doc_start.numel(), device=doc_start.device, dtype=doc_start.dtype)
    ok = (doc_start >= 0) & (doc_start <= pos)
    if doc_start.numel() > 1:
        ok[1:] &= doc_start[1:] >= doc_start[:-1]
    if not bool(ok.all()):
        raise ValueError("doc_start must satisfy 0 <= doc_start[t] <= t and must not decrease")


def decode_workspace_bytes(B: int, H: int, D: int, n_rows: int, nsplit: int = 0) -> int:
    return int(_lib.load().daisy_decode_workspace_bytes(B, H, D, n_rows, nsplit))


def decode_attention(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                     k_rows: Optional[torch.Tensor], v_rows: Optional[torch.Tensor], *,
                     n_rows: int, new_idx: int, write_back: bool,
                     scale: float = ATTN_SCALE,
                     cos_row: Optional[torch.Tensor] = None, sin_row: Optional[torch.Tensor] = None,
                     out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
                     nsplit: int = 0) -> torch.Tensor:
    """One decode step for every (batch, head).

    ``q``, ``k_new``, ``v_new``: bf16 ``[B, H, D]`` (any batch/head strides).
    ``k_rows``/``v_rows``: bf16 tensors addressed as ``[B, H, rows, D]`` through
    their strides (dims 0, 1, 2); logical rows ``0..n_rows-1`` are attended,
    except that row ``new_idx`` is taken from ``k_new``/``v_new`` (after RoPE
    with ``cos_row``/``sin_row``) and stored back when ``write_back``.
    Returns ``o`` bf16 ``[B, H, D]``.
    """
    dev = _lib.require_gpu(q, k_new, v_new, k_rows, v_rows, cos_row, sin_row, out, workspace)
    for name, t in (("q", q), ("k_new", k_new), ("v_new", v_new)):
        _check_bf16(name, t, 3)
    B, H, D = q.shape
    if k_new.shape != q.shape or v_new.shape != q.shape:
        raise ValueError("q, k_new, v_new must all be [B, H, D]")
    if k_rows is not None:
        _check_bf16("k_rows", k_rows, 4)
        _check_bf16("v_rows", v_rows, 4)
    if out is None:
        out = torch.empty((B, H, D), dtype=torch.bfloat16, device=dev)
    else:
        _check_bf16("out", out, 3)
    lib = _lib.load()
    need = int(lib.daisy_decode_workspace_bytes(B, H, D, n_rows, nsplit))
    if need > 0 and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with _lib.on_device(dev):
        rc = lib.daisy_decode_fwd(
            q.data_ptr(), _lib.strides(q, (0, 1)),
            k_new.data_ptr(), _lib.strides(k_new, (0, 1)),
            v_new.data_ptr(), _lib.strides(v_new, (0, 1)),
            _lib.ptr(k_rows), None if k_rows is None else _lib.strides(k_rows, (0, 1, 2)),
            _lib.ptr(v_rows), None if v_rows is None else _lib.strides(v_rows, (0, 1, 2)),
            _lib.ptr(cos_row), _lib.ptr(sin_row),
            out.data_ptr(), _lib.strides(out, (0, 1)),
            B, H, D, int(n_rows), int(new_idx), 1 if write_back else 0,
            float(scale), int(nsplit),
            _lib.ptr(workspace), ws_bytes, _lib.current_stream(dev))
    _lib.check(rc, "daisy_decode_fwd")
    return out


def decode_attention_at(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                        k_ring: torch.Tensor, v_ring: torch.Tensor, pos: torch.Tensor, *,
                        scale: float = ATTN_SCALE, out: Optional[torch.Tensor] = None,
                        workspace: Optional[torch.Tensor] = None, nsplit: int = 0) -> torch.Tensor:
    """``decode_attention`` over a ring cache with the position in device memory.

    ``k_ring``/``v_ring``: bf16 ``[B, H, W, D]`` (slot order); ``pos``: one-element int32 device tensor
    holding ``t``, the number of positions already in the ring.  The kernel reads ``t`` when it
    runs, attends the ``min(t + 1, W)`` live rows and writes the new row (``k_new``, ``v_new``, already
    rotated) to slot ``t % W``; the launch can therefore be recorded in a HIP graph and replayed
    while the caller increments ``pos``.  Returns ``o`` bf16 ``[B, H, D]``.
    """
    dev = _lib.require_gpu(q, k_new, v_new, k_ring, v_ring, pos, out, workspace)
    for name, t in (("q", q), ("k_new", k_new), ("v_new", v_new)):
        _check_bf16(name, t, 3)
    _check_bf16("k_ring", k_ring, 4)
    _check_bf16("v_ring", v_ring, 4)
    B, H, D = q.shape
    if k_new.shape != q.shape or v_new.shape != q.shape:
        raise ValueError("q, k_new, v_new must all be [B, H, D]")
    W = k_ring.shape[2]
    if k_ring.shape != (B, H, W, D) or v_ring.shape != k_ring.shape:
        raise ValueError(f"k_ring, v_ring must be [B, H, W, D] = [{B}, {H}, W, {D}], got {tuple(k_ring.shape)}, {tuple(v_ring.shape)}")
    if pos.dtype != torch.int32 or pos.numel() != 1:
        raise ValueError("pos must be a one-element int32 tensor")
    if out is None:
        out = torch.empty((B, H, D), dtype=torch.bfloat16, device=dev)
    else:
        _check_bf16("out", out, 3)
    lib = _lib.load()
    need = int(lib.daisy_decode_workspace_bytes(B, H, D, W, nsplit))
    if need > 0 and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with _lib.on_device(dev):
        rc = lib.daisy_decode_fwd_at(
            q.data_ptr(), _lib.strides(q, (0, 1)),
            k_new.data_ptr(), _lib.strides(k_new, (0, 1)),
            v_new.data_ptr(), _lib.strides(v_new, (0, 1)),
            k_ring.data_ptr(), _lib.strides(k_ring, (0, 1, 2)),
            v_ring.data_ptr(), _lib.strides(v_ring, (0, 1, 2)),
            out.data_ptr(), _lib.strides(out, (0, 1)),
            B, H, D, int(W), pos.data_ptr(), float(scale), int(nsplit),
            _lib.ptr(workspace), ws_bytes, _lib.current_stream(dev))
    _lib.check(rc, "daisy_decode_fwd_at")
    return out


def attn_step(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_ring: torch.Tensor, v_ring: torch.Tensor,
              pos: Union[int, torch.Tensor], *, cos: torch.Tensor, sin: torch.Tensor, eps: float,
              ve: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
              scale: float = ATTN_SCALE, out: Optional[torch.Tensor] = None,
              workspace: Optional[torch.Tensor] = None, nsplit: int = 0,
              status: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The attention part of one decode step in one launch (``daisy_attn_step_fwd``).

    ``q``, ``k``, ``v``: the new token's rows of the QKV projection output, bf16 ``[B, H, D]`` views;
    the kernel normalises them, rotates q and k with row ``pos`` of ``cos``/``sin`` (fp32
    ``[rows, D/2]``), mixes ``v`` with ``ve [B, H, D]`` through ``gate`` (one fp32), writes the new rows
    into slot ``pos % W`` of ``k_ring``/``v_ring [B, H, W, D]`` (bf16 or fp16) and attends the live rows.  ``pos`` is an
    int or a one-element int32 device tensor (read when the kernel runs).  Returns ``o [B, H, D]``.

    ``status``: one-element int32 device tensor.  A device position past the rotary tables cannot
    be refused on the host; the kernel then writes NaN outputs and raises bit
    ``_lib.STATUS_POSITION_PAST_TABLES`` in ``status`` (see ``raise_for_status``).
    """
    pos_dev = pos if isinstance(pos, torch.Tensor) else None
    dev = _lib.require_gpu(q, k, v, k_ring, v_ring, cos, sin, ve, gate, pos_dev, out, workspace, status)
    _check_status(status)
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_bf16(name, t, 3)
    if k_ring.dtype == torch.float16 and v_ring.dtype == torch.float16 and k_ring.dim() == 4 and k_ring.stride(-1) == 1 \
            and v_ring.stride(-1) == 1:
        ring_f16 = True       # the reference generator's default cache dtype
    else:
        ring_f16 = False
        _check_bf16("k_ring", k_ring, 4)
        _check_bf16("v_ring", v_ring, 4)
    B, H, D = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k, v must all be [B, H, D]")
    W = k_ring.shape[2]
    if k_ring.shape != (B, H, W, D) or v_ring.shape != k_ring.shape:
        raise ValueError(f"k_ring, v_ring must be [{B}, {H}, W, {D}], got {tuple(k_ring.shape)}, {tuple(v_ring.shape)}")
    for name, t in (("cos", cos), ("sin", sin)):
        if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != D // 2 or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous fp32 [rows, {D // 2}] table, got {tuple(t.shape)} {t.dtype}")
    if pos_dev is not None:
        if pos_dev.dtype != torch.int32 or pos_dev.numel() != 1:
            raise ValueError("a device position must be a one-element int32 tensor")
        live = W
    else:
        torch._assert(0 <= pos < cos.shape[0], f"Rotary buffers too small {cos.shape[0]} < {pos + 1}")
        live = min(int(pos) + 1, W)
    if (ve is None) != (gate is None):
        raise ValueError("ve and gate must be given together")
    if ve is not None:
        _check_bf16("ve", ve, 3)
        if ve.shape != q.shape or gate.dtype != torch.float32 or gate.numel() != 1:
            raise ValueError("ve must be [B, H, D] and gate a one-element fp32 tensor")
    if out is None:
        out = torch.empty((B, H, D), dtype=torch.bfloat16, device=dev)
    else:
        _check_bf16("out", out, 3)
    lib = _lib.load()
    need = int(lib.daisy_decode_workspace_bytes(B, H, D, live, nsplit))
    if need > 0 and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    d2 = (0, 1)
    with _lib.on_device(dev):
        rc = lib.daisy_attn_step_fwd(
            q.data_ptr(), _lib.strides(q, d2), k.data_ptr(), _lib.strides(k, d2), v.data_ptr(), _lib.strides(v, d2),
            _lib.ptr(ve), None if ve is None else _lib.strides(ve, d2), _lib.ptr(gate),
            cos.data_ptr(), sin.data_ptr(), int(cos.shape[0]),
            0 if pos_dev is not None else int(pos), _lib.ptr(pos_dev), _lib.ptr(status), float(eps),
            k_ring.data_ptr(), _lib.strides(k_ring, (0, 1, 2)), v_ring.data_ptr(), _lib.strides(v_ring, (0, 1, 2)),
            1 if ring_f16 else 0,
            out.data_ptr(), _lib.strides(out, d2), B, H, D, int(W), float(scale), int(nsplit),
            _lib.ptr(workspace), ws_bytes, _lib.current_stream(dev))
    _lib.check(rc, "daisy_attn_step_fwd")
    return out


def attn_layer_step(x: torch.Tensor, w_qkv: torch.Tensor, w_out: torch.Tensor, k_ring: torch.Tensor,
                    v_ring: torch.Tensor, pos: Union[int, torch.Tensor], *, cos: torch.Tensor, sin: torch.Tensor,
                    eps: float, ve: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                    scale: float = ATTN_SCALE, nsplit: int = 0, status: Optional[torch.Tensor] = None,
                    workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One decode step of an attention layer in one call (``daisy_attn_layer_step_fwd``): QKV projection of
    ``x [B, dim]`` (or ``[B, 1, dim]``) with ``w_qkv [3*H*D, dim]``, the one-launch attention step of ``attn_step`` on
    the rings ``[B, H, W, D]``, output projection with ``w_out [dim, H*D]``.  bf16 throughout (the rings may be fp16),
    ``B`` at most ``_lib.LINEAR_MAX_ROWS``.  Returns ``y`` shaped like ``x``.  Same results as ``linear_rows``,
    ``attn_step``, ``linear_rows`` one after the other; what it saves is the host's time between the launches."""
    pos_dev = pos if isinstance(pos, torch.Tensor) else None
    dev = _lib.require_gpu(x, w_qkv, w_out, k_ring, v_ring, cos, sin, ve, gate, pos_dev, status, workspace)
    _check_status(status)
    if x.dtype != torch.bfloat16 or w_qkv.dtype != torch.bfloat16 or w_out.dtype != torch.bfloat16:
        raise TypeError("attn_layer_step: x, w_qkv and w_out must be bf16")
    if k_ring.dtype != v_ring.dtype or k_ring.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"attn_layer_step: the rings must both be bf16 or both fp16, got {k_ring.dtype}, {v_ring.dtype}")
    if k_ring.dim() != 4 or v_ring.shape != k_ring.shape or k_ring.stride(3) != 1 or v_ring.stride(3) != 1:
        raise ValueError("attn_layer_step: k_ring, v_ring must be [B, H, W, D] with a contiguous last dim")
    B, H, W, D = k_ring.shape
    dim = x.shape[-1]
    if x.numel() != B * dim or w_qkv.shape != (3 * H * D, dim) or w_out.shape != (dim, H * D):
        raise ValueError(f"attn_layer_step: x {tuple(x.shape)}, w_qkv {tuple(w_qkv.shape)}, w_out {tuple(w_out.shape)} do not "
                         f"fit rings of {B} x {H} x {D}")
    if not (x.is_contiguous() and w_qkv.stride(1) == 1 and w_out.stride(1) == 1):
        raise ValueError("attn_layer_step: x must be contiguous and the weights' last dims contiguous")
    for name, t in (("cos", cos), ("sin", sin)):
        if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != D // 2 or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous fp32 [rows, {D // 2}] table, got {tuple(t.shape)} {t.dtype}")
    if pos_dev is not None:
        if pos_dev.dtype != torch.int32 or pos_dev.numel() != 1:
            raise ValueError("a device position must be a one-element int32 tensor")
    else:
        torch._assert(0 <= pos < cos.shape[0], f"Rotary buffers too small {cos.shape[0]} < {pos + 1}")
    if (ve is None) != (gate is None):
        raise ValueError("ve and gate must be given together")
    ve_strides = None
    if ve is not None:
        if ve.dtype != torch.bfloat16 or ve.shape != (B, H, D) or ve.stride(2) != 1:
            raise ValueError(f"ve must be bf16 [{B}, {H}, {D}] with a contiguous last dim, got {tuple(ve.shape)} {ve.dtype}")
        if gate.dtype != torch.float32 or gate.numel() != 1:
            raise ValueError("gate must be a one-element fp32 tensor")
        ve_strides = _lib.strides(ve, (0, 1))
    lib = _lib.load()
    need = int(lib.daisy_attn_layer_step_workspace_bytes(B, H, D, W, nsplit))
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    y = torch.empty_like(x)
    with _lib.on_device(dev):
        rc = lib.daisy_attn_layer_step_fwd(
            x.data_ptr(), dim, w_qkv.data_ptr(), w_qkv.stride(0), w_out.data_ptr(), w_out.stride(0),
            _lib.ptr(ve), ve_strides, _lib.ptr(gate), cos.data_ptr(), sin.data_ptr(), int(cos.shape[0]),
            0 if pos_dev is not None else int(pos), _lib.ptr(pos_dev), _lib.ptr(status), float(eps),
            k_ring.data_ptr(), _lib.strides(k_ring, (0, 1, 2)), v_ring.data_ptr(), _lib.strides(v_ring, (0, 1, 2)),
            1 if k_ring.dtype == torch.float16 else 0, y.data_ptr(), dim, B, H, D, dim, W, float(scale), int(nsplit),
            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _lib.current_stream(dev))
    _lib.check(rc, "daisy_attn_layer_step_fwd")
    return y


def _check_status(status: Optional[torch.Tensor]) -> None:
    if status is not None and (status.dtype != torch.int32 or status.numel() != 1):
        raise ValueError("status must be a one-element int32 tensor")


def raise_for_status(status: torch.Tensor) -> None:
    """Reads a status word (synchronises) and raises what the kernels reported in it."""
    bits = int(status.item())
    if bits & _lib.STATUS_POSITION_PAST_TABLES:
        raise RuntimeError("a decode step ran at a position past the rotary tables (Rotary buffers too small); "
                           "its outputs are NaN")


def kda_workspace_bytes(B: int, T: int, H: int, Dk: int, Dv: int, chunk: int = 64) -> int:
    return int(_lib.load().daisy_kda_workspace_bytes(B, T, H, Dk, Dv, chunk))


def _check_cu_seqlens(cu_seqlens: torch.Tensor, B: int) -> int:
    """Validates what the host can see of packed-sequence bounds; returns the sequence count."""
    if B != 1:
        raise ValueError("cu_seqlens needs batch size 1 (sequences packed along T)")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2 or not cu_seqlens.is_contiguous():
        raise ValueError("cu_seqlens must be a contiguous int32 [n_seq + 1] tensor")
    return cu_seqlens.numel() - 1


def _kda_inputs(q, k, v, g, beta, initial_state, n_states, scale, fresh_state_copy=True):
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_bf16(name, t, 4)
    B, T, H, Dk = q.shape
    Dv = v.shape[-1]
    if k.shape != q.shape or g.shape != q.shape or v.shape[:3] != q.shape[:3] or beta.shape != (B, T, H):
        raise ValueError("kda: expected q,k,g [B,T,H,Dk], v [B,T,H,Dv], beta [B,T,H]")
    if g.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"g must be fp32 or bf16, got {g.dtype}")
    q, k, v, g = q.contiguous(), k.contiguous(), v.contiguous(), g.contiguous()
    beta = beta.to(torch.float32).contiguous()
    if scale is None:
        scale = Dk ** -0.5
    if initial_state is not None:
        if initial_state.shape != (n_states, H, Dk, Dv):
            raise ValueError(f"initial_state must be [{n_states},H,Dk,Dv], got {tuple(initial_state.shape)}")
        if fresh_state_copy:
            initial_state = initial_state.to(torch.float32).contiguous()
    return q, k, v, g, beta, initial_state, scale


def kda_chunk_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, beta: torch.Tensor, *,
                  scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                  output_final_state: bool = False, use_qk_l2norm_in_kernel: bool = True,
                  l2_eps: float = 1e-6, chunk: int = 64, cu_seqlens: Optional[torch.Tensor] = None,
                  workspace: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Chunked KDA forward; see ``daisy_kda_chunk_fwd`` / ``daisy_kda_chunk_varlen_fwd`` in ``include/daisy_hip.h``.

    ``cu_seqlens`` (int32 ``[N + 1]`` on the GPU, from 0 to T, non-decreasing): the batch is 1 and
    holds N sequences packed along T, each with its own state ``[N, H, Dk, Dv]``.  The kernels read
    the bounds on the device; the host never does, so the call does not synchronise.
    """
    dev = _lib.require_gpu(q, k, v, g, beta, initial_state, workspace, cu_seqlens)
    B, T, H, Dk = q.shape
    Dv = v.shape[-1]
    n_seq = _check_cu_seqlens(cu_seqlens, B) if cu_seqlens is not None else 0
    n_states = n_seq if n_seq else B
    q, k, v, g, beta, initial_state, scale = _kda_inputs(q, k, v, g, beta, initial_state, n_states, scale)
    # rows that belong to no sequence (bounds that stop short of T) are not written by the kernels
    o = (torch.zeros if n_seq else torch.empty)((B, T, H, Dv), dtype=torch.bfloat16, device=dev)
    final = torch.empty((n_states, H, Dk, Dv), dtype=torch.float32, device=dev) if output_final_state else None
    lib = _lib.load()
    if n_seq:
        need = int(lib.daisy_kda_varlen_workspace_bytes(T, n_seq, H, Dk, Dv, chunk))
    else:
        need = int(lib.daisy_kda_workspace_bytes(B, T, H, Dk, Dv, chunk))
    if need > 0 and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), 1 if g.dtype == torch.bfloat16 else 0, beta.data_ptr())
    tail = (int(chunk), float(scale), 1 if use_qk_l2norm_in_kernel else 0, float(l2_eps),
            _lib.ptr(workspace), ws_bytes, _lib.current_stream(dev))
    with _lib.on_device(dev):
        if n_seq:
            rc = lib.daisy_kda_chunk_varlen_fwd(*head, cu_seqlens.data_ptr(), n_seq, _lib.ptr(initial_state), o.data_ptr(),
                                                _lib.ptr(final), T, H, Dk, Dv, *tail)
        else:
            rc = lib.daisy_kda_chunk_fwd(*head, _lib.ptr(initial_state), o.data_ptr(), _lib.ptr(final), B, T, H, Dk, Dv, *tail)
    _lib.check(rc, "daisy_kda_chunk_fwd")
    return o, final


def kda_recurrent_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, beta: torch.Tensor, *,
                      scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                      output_final_state: bool = True, use_qk_l2norm_in_kernel: bool = True,
                      l2_eps: float = 1e-6, inplace_state: bool = False,
                      cu_seqlens: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Token-by-token KDA with the state in registers; see ``daisy_kda_recurrent_fwd``.

    With ``inplace_state`` the final state overwrites ``initial_state`` (which must then be a
    contiguous fp32 ``[B, H, Dk, Dv]`` tensor) and is returned as such -- the decode loop's mode.
    ``cu_seqlens``: packed sequences as in ``kda_chunk_fwd``.
    """
    dev = _lib.require_gpu(q, k, v, g, beta, initial_state, cu_seqlens)
    B, T, H, Dk = q.shape
    Dv = v.shape[-1]
    n_seq = _check_cu_seqlens(cu_seqlens, B) if cu_seqlens is not None else 0
    n_states = n_seq if n_seq else B
    if inplace_state:
        if initial_state is None:
            raise ValueError("inplace_state needs an initial_state")
        if initial_state.dtype != torch.float32 or not initial_state.is_contiguous():
            raise ValueError("inplace_state needs a contiguous fp32 initial_state")
    q, k, v, g, beta, initial_state, scale = _kda_inputs(q, k, v, g, beta, initial_state, n_states, scale,
                                                         fresh_state_copy=not inplace_state)
    o = (torch.zeros if n_seq else torch.empty)((B, T, H, Dv), dtype=torch.bfloat16, device=dev)
    if inplace_state:
        final = initial_state
    else:
        final = torch.empty((n_states, H, Dk, Dv), dtype=torch.float32, device=dev) if output_final_state else None
    lib = _lib.load()
    head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), 1 if g.dtype == torch.bfloat16 else 0, beta.data_ptr())
    tail = (float(scale), 1 if use_qk_l2norm_in_kernel else 0, float(l2_eps), _lib.current_stream(dev))
    with _lib.on_device(dev):
        if n_seq:
            rc = lib.daisy_kda_recurrent_varlen_fwd(*head, cu_seqlens.data_ptr(), n_seq, _lib.ptr(initial_state), o.data_ptr(),
                                                    _lib.ptr(final), T, H, Dk, Dv, *tail)
        else:
            rc = lib.daisy_kda_recurrent_fwd(*head, _lib.ptr(initial_state), o.data_ptr(), _lib.ptr(final), B, T, H, Dk, Dv, *tail)
    _lib.check(rc, "daisy_kda_recurrent_fwd")
    return o, final


def kda_gate_fwd(g: torch.Tensor, A_log: torch.Tensor, head_k_dim: int,
                 g_bias: Optional[torch.Tensor] = None, beta: float = 1.0, threshold: float = 20.0) -> torch.Tensor:
    """``-exp(A_log[h]) * softplus(g + bias)``; ``g [..., H*Dk]`` -> ``[..., H, Dk]`` in ``g.dtype``."""
    dev = _lib.require_gpu(g, A_log, g_bias)
    if g.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"g must be fp32 or bf16, got {g.dtype}")
    last = g.shape[-1]
    if last % head_k_dim != 0:
        raise RuntimeError("last dim must be divisible by head_k_dim")
    H = last // head_k_dim
    if A_log.numel() != H:
        raise RuntimeError(f"A_log must be shape [H] or [1,1,H,1]; got {tuple(A_log.shape)} with H={H}")
    a = A_log.detach().reshape(H).to(device=dev, dtype=torch.float32).contiguous()
    bias = None
    if g_bias is not None:
        b = g_bias.detach().to(device=dev, dtype=torch.float32)
        if b.numel() == H * head_k_dim:
            bias = b.reshape(H, head_k_dim).contiguous()
        elif b.numel() == H:
            bias = b.reshape(H, 1).expand(H, head_k_dim).contiguous()
        else:
            raise RuntimeError(f"g_bias must be one of [(H*D,), (H,D), (1,1,H,D), (H,)]; got {tuple(b.shape)}")
    gc = g.contiguous()
    out = torch.empty((*g.shape[:-1], H, head_k_dim), dtype=g.dtype, device=dev)
    rows = gc.numel() // last
    lib = _lib.load()
    with _lib.on_device(dev):
        rc = lib.daisy_kda_gate_fwd(gc.data_ptr(), a.data_ptr(), _lib.ptr(bias), out.data_ptr(),
                                    rows, H, head_k_dim, 1 if g.dtype == torch.bfloat16 else 0,
                                    float(beta), float(threshold), _lib.current_stream(dev))
    _lib.check(rc, "daisy_kda_gate_fwd")
    return out


def linear_rows_ok(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether ``linear_rows`` takes this pair: bf16 on a GPU, at most ``_lib.LINEAR_MAX_ROWS`` rows of ``x``,
    rows of both starting on 16-byte boundaries."""
    if not (x.is_cuda and weight.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16):
        return False
    if weight.dim() != 2 or x.dim() < 1 or x.shape[-1] != weight.shape[1] or weight.shape[1] % 8 != 0:
        return False
    rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
    if not 1 <= rows <= _lib.LINEAR_MAX_ROWS:
        return False
    return weight.stride(1) == 1 and weight.stride(0) % 8 == 0 and weight.data_ptr() % 16 == 0


def linear_rows(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``F.linear(x, weight)`` for the few activation rows of a decode step (``daisy_linear_rows_fwd``):
    ``x [..., K]`` bf16 with at most ``_lib.LINEAR_MAX_ROWS`` rows in all, ``weight [N, K]`` bf16 (rows may be
    strided); returns ``[..., N]`` bf16.  Reads the weights once; fp32 accumulation, one rounding."""
    dev = _lib.require_gpu(x, weight, out)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError(f"linear_rows: x and weight must be bf16, got {x.dtype}, {weight.dtype}")
    if weight.dim() != 2 or x.dim() < 1 or x.shape[-1] != weight.shape[1]:
        raise ValueError(f"linear_rows: x [..., K] and weight [N, K] do not fit: {tuple(x.shape)}, {tuple(weight.shape)}")
    if weight.stride(1) != 1:
        raise ValueError("linear_rows: the weight's last dim must be contiguous")
    N, K = weight.shape
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1 or (x2.size(0) > 1 and x2.stride(0) % 8 != 0) or x2.data_ptr() % 16 != 0:
        x2 = x2.contiguous()
    M = x2.size(0)
    if out is None:
        out = torch.empty(*x.shape[:-1], N, dtype=torch.bfloat16, device=dev)
    elif out.dtype != torch.bfloat16 or out.shape != (*x.shape[:-1], N) or not out.is_contiguous():
        raise ValueError(f"linear_rows: out must be a contiguous bf16 {(*x.shape[:-1], N)} tensor")
    lib = _lib.load()
    with _lib.on_device(dev):
        rc = lib.daisy_linear_rows_fwd(x2.data_ptr(), x2.stride(0) if M > 1 else K, weight.data_ptr(), weight.stride(0),
                                       out.data_ptr(), N, M, N, K, _lib.current_stream(dev))
    _lib.check(rc, "daisy_linear_rows_fwd")
    return out


def qkv_prep(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, eps: float,
             cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
             pos0: Union[int, torch.Tensor] = 0,
             ve: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
             q_out: Optional[torch.Tensor] = None, k_out: Optional[torch.Tensor] = None,
             v_out: Optional[torch.Tensor] = None, status: Optional[torch.Tensor] = None
             ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """RMS norm of q, k, v + RoPE of q, k at rows ``pos0 + t`` + ``gate*v + (1-gate)*ve`` in one pass.

    ``q``, ``k``, ``v`` (and ``ve``) are bf16 ``[B, T, H, D]`` tensors or views with a
    contiguous last dim; ``gate`` is a one-element fp32 tensor holding the (bf16-rounded)
    sigmoid of the gate logit.  Outputs default to new contiguous ``[B, T, H, D]`` tensors;
    any strided bf16 ``[B, T, H, D]`` view may be passed instead.

    ``pos0`` may be a one-element int32 device tensor: the kernel then reads the position when
    it runs (a launch recorded in a HIP graph follows the tensor's value from replay to replay);
    ``pos0 + T`` beyond the tables cannot be refused here: the kernel then writes NaN for the rotated
    outputs and raises ``_lib.STATUS_POSITION_PAST_TABLES`` in ``status`` (one-element int32 tensor).
    """
    pos_dev = pos0 if isinstance(pos0, torch.Tensor) else None
    if pos_dev is not None:
        if pos_dev.dtype != torch.int32 or pos_dev.numel() != 1:
            raise ValueError("a device position must be a one-element int32 tensor")
        if cos is None:
            raise ValueError("a device position needs the rotary tables")
        pos0 = 0
    dev = _lib.require_gpu(q, k, v, ve, gate, cos, sin, q_out, k_out, v_out, pos_dev, status)
    _check_status(status)
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_bf16(name, t, 4)
    B, T, H, D = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"q, k, v shapes differ: {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    if (cos is None) != (sin is None):
        raise ValueError("cos and sin must be given together")
    if cos is not None:
        for name, t in (("cos", cos), ("sin", sin)):
            if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != D // 2 or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous fp32 [rows, {D // 2}] table, got {tuple(t.shape)} {t.dtype}")
            torch._assert(pos0 + T <= t.shape[0], f"Rotary buffers too small {t.shape[0]} < {pos0 + T}")
    if (ve is None) != (gate is None):
        raise ValueError("ve and gate must be given together")
    if ve is not None:
        _check_bf16("ve", ve, 4)
        if ve.shape != q.shape:
            raise ValueError(f"ve must have shape {tuple(q.shape)}, got {tuple(ve.shape)}")
        if gate.dtype != torch.float32 or gate.numel() != 1:
            raise ValueError("gate must be a one-element fp32 tensor")
    outs = []
    for name, t in (("q_out", q_out), ("k_out", k_out), ("v_out", v_out)):
        if t is None:
            t = torch.empty((B, T, H, D), dtype=torch.bfloat16, device=dev)
        else:
            _check_bf16(name, t, 4)
            if t.shape != q.shape:
                raise ValueError(f"{name} must have shape {tuple(q.shape)}, got {tuple(t.shape)}")
        outs.append(t)
    qo, ko, vo = outs
    d3 = (0, 1, 2)
    lib = _lib.load()
    ins = (q.data_ptr(), _lib.strides(q, d3), k.data_ptr(), _lib.strides(k, d3), v.data_ptr(), _lib.strides(v, d3),
           _lib.ptr(ve), None if ve is None else _lib.strides(ve, d3), _lib.ptr(gate), _lib.ptr(cos), _lib.ptr(sin))
    outs = (qo.data_ptr(), _lib.strides(qo, d3), ko.data_ptr(), _lib.strides(ko, d3), vo.data_ptr(), _lib.strides(vo, d3),
            B, T, H, D, float(eps))
    with _lib.on_device(dev):
        if pos_dev is None:
            rc = lib.daisy_qkv_prep_fwd(*ins, int(pos0), *outs, _lib.current_stream(dev))
        else:
            rc = lib.daisy_qkv_prep_fwd_at(*ins, pos_dev.data_ptr(), int(cos.shape[0]), _lib.ptr(status), *outs,
                                           _lib.current_stream(dev))
    _lib.check(rc, "daisy_qkv_prep_fwd")
    return qo, ko, vo


def short_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               cache: Optional[torch.Tensor] = None, output_final_state: bool = False,
               activation: Optional[str] = "silu", inplace_cache: bool = False,
               cu_seqlens: Optional[torch.Tensor] = None
               ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Depthwise causal convolution over time + SiLU for ``x [B, T, C]`` bf16 (``daisy_short_conv_fwd``).

    ``weight [C, 1, K]`` or ``[C, K]``; ``cache [B, C, K]`` holds the last K inputs of the sequence
    so far.  Returns ``(y [B, T, C], new cache or None)``.  ``inplace_cache``: the new window is
    written into ``cache`` itself (bf16, contiguous, ``T <= 32``: decode steps) and ``cache`` is returned.
    ``cu_seqlens`` (int32 ``[N + 1]`` on the GPU): ``B == 1`` and N sequences are packed along T; no tap
    reaches across the start of its sequence and the windows are ``[N, C, K]`` (``daisy_short_conv_varlen_fwd``).
    """
    dev = _lib.require_gpu(x, weight, bias, cache, cu_seqlens)
    _check_bf16("x", x, 3)
    B, T, C = x.shape
    n_seq = _check_cu_seqlens(cu_seqlens, B) if cu_seqlens is not None else 0
    n_win = n_seq if n_seq else B
    w = weight.reshape(C, -1)
    K = w.shape[1]
    if w.dtype != torch.bfloat16 or (bias is not None and bias.dtype != torch.bfloat16):
        raise TypeError("short_conv: weight and bias must be bf16")
    if activation not in (None, "silu"):
        raise ValueError(f"short_conv: activation {activation!r} not supported")
    if x.stride(2) != 1:
        x = x.contiguous()
    w = w.contiguous()
    if cache is not None:
        if cache.shape != (n_win, C, K):
            raise ValueError(f"short_conv: cache must be [{n_win}, {C}, {K}], got {tuple(cache.shape)}")
        if inplace_cache and (cache.dtype != torch.bfloat16 or not cache.is_contiguous()):
            raise ValueError("short_conv: a window updated in place must be a contiguous bf16 tensor")
        cache = cache.to(torch.bfloat16).contiguous()
    elif inplace_cache:
        raise ValueError("short_conv: inplace_cache needs a cache")
    y = torch.empty(B, T, C, dtype=torch.bfloat16, device=dev)
    if inplace_cache:
        new_cache = cache
    else:
        new_cache = torch.empty(n_win, C, K, dtype=torch.bfloat16, device=dev) if output_final_state else None
    lib = _lib.load()
    if n_seq:
        if inplace_cache:
            raise ValueError("short_conv: inplace_cache does not combine with cu_seqlens")
        if bias is not None:
            bias = bias.contiguous()
        with _lib.on_device(dev):
            rc = lib.daisy_short_conv_varlen_fwd(x.data_ptr(), x.stride(1), w.data_ptr(), _lib.ptr(bias),
                                                 cu_seqlens.data_ptr(), n_seq, _lib.ptr(cache),
                                                 y.data_ptr(), y.stride(1), _lib.ptr(new_cache),
                                                 T, C, K, 1 if activation == "silu" else 0, _lib.current_stream(dev))
        _lib.check(rc, "daisy_short_conv_varlen_fwd")
        return y, new_cache
    with _lib.on_device(dev):
        rc = lib.daisy_short_conv_fwd(x.data_ptr(), _lib.strides(x, (0, 1)), w.data_ptr(), _lib.ptr(bias), _lib.ptr(cache),
                                      y.data_ptr(), _lib.strides(y, (0, 1)), _lib.ptr(new_cache),
                                      B, T, C, K, 1 if activation == "silu" else 0, _lib.current_stream(dev))
    _lib.check(rc, "daisy_short_conv_fwd")
    return y, new_cache


def gated_rmsnorm(x: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """``x * rsqrt(mean(x^2) + eps) * weight * sigmoid(gate)`` over the last dim (64 or 128), bf16."""
    dev = _lib.require_gpu(x, gate, weight)
    if x.dtype != torch.bfloat16 or gate.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("gated_rmsnorm: x, gate and weight must be bf16")
    if gate.shape != x.shape or weight.numel() != x.shape[-1]:
        raise ValueError(f"gated_rmsnorm: shapes {tuple(x.shape)}, {tuple(gate.shape)}, {tuple(weight.shape)} do not match")
    xc, gc, wc = x.contiguous(), gate.contiguous(), weight.contiguous()
    out = torch.empty_like(xc)
    D = x.shape[-1]
    lib = _lib.load()
    with _lib.on_device(dev):
        rc = lib.daisy_gated_rmsnorm_fwd(xc.data_ptr(), gc.data_ptr(), wc.data_ptr(), out.data_ptr(),
                                         xc.numel() // D, D, float(eps), _lib.current_stream(dev))
    _lib.check(rc, "daisy_gated_rmsnorm_fwd")
    return out
