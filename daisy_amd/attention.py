"""Drop-in ``CausalSelfAttention`` / ``Rotary`` backed by the gfx950 kernels.

Mirrors models/daisy/attention.py of the reference: same constructor, same
state-dict keys (``qkvo_w``, optional ``g_ve``), same ``forward`` / ``prefill`` /
``step`` / ``reset_history`` signatures, shapes and dtypes.  The QKV and output
projections and the weightless RMS norms stay PyTorch library calls; RoPE, the
mask and the attention itself run in ``libdaisy_hip.so``.  Inference only: the
kernels have no backward.

Masks.  The reference passes a dense additive ``[1, 1, T, T]`` mask built by
``build_attn_mask`` (models/daisy/daisy_core.py:53-69).  Here the mask is the
light descriptor ``WindowMask(window, doc_start)``; ``build_window_mask`` makes
one from token ids.  A dense reference mask is still accepted and converted
(each row must allow one contiguous run of keys ending at the query).
"""
from __future__ import annotations

import os
import weakref
from dataclasses import dataclass
from typing import Optional, Tuple, Union

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import ops
from .functional import NORM_EPS_BF16, init_linear, norm
from .kv_cache import RingContext


@dataclass
class WindowMask:
    """``0 <= q - k < window`` and ``k >= doc_start[q]``.

    ``window``: keys visible per query including itself (``None`` = unlimited).
    ``doc_start``: int32 ``[T]`` on the GPU, first position of each query's
    document, or ``None`` for a single document; ``0 <= doc_start[q] <= q`` and
    non-decreasing (the attention kernel skips key tiles by it).
    ``kv_out``: optional ``(k, v)`` pair of bf16 ``[B, T, H, D]`` views that receive the keys
    (normalised, rotated) and values (normalised, mixed) of the call the mask is passed to, e.g.
    slots of a ring cache, so that no copy into the cache follows.  The model glue sets it per
    layer; a reference-style ``Block`` passes the descriptor through untouched.
    """
    window: Optional[int]
    doc_start: Optional[Tensor] = None
    kv_out: Optional[Tuple[Tensor, Tensor]] = None


def doc_start_from_ids(input_seq: Tensor, eos_token_id: int) -> Tensor:
    """int32 ``[T]``: position of the latest EOS at or before each token (0 if none).

    The reference numbers documents with ``cumsum(ids == eos)``
    (models/daisy/daisy_core.py:60), so an EOS token opens its own document.
    """
    ids = input_seq.reshape(-1)
    pos = torch.arange(ids.numel(), device=ids.device, dtype=torch.int32)
    marks = torch.where(ids == eos_token_id, pos, torch.zeros_like(pos))
    return torch.cummax(marks, dim=0).values.to(torch.int32).contiguous()


def build_window_mask(input_seq: Tensor, window_size: Optional[int], eos_token_id: Optional[int]) -> WindowMask:
    """Descriptor equivalent of the reference's ``build_attn_mask`` (no T x T tensor)."""
    ds = None if eos_token_id is None else doc_start_from_ids(input_seq, eos_token_id)
    return WindowMask(window_size, ds)


def build_block_window_masks(input_seq: Tensor, sliding_window_num_blocks, num_layers: int,
                             eos_token_id: int, block: int = 128):
    """Per-layer descriptors equal to the reference's training-time block masks
    (``DaisyCore.create_blockmasks``, models/daisy/daisy_core.py:182-229).

    There the window is counted in key blocks of ``block`` tokens: a query block sees its own
    block and the ``w - 1`` blocks before it, element-wise restricted to ``k <= q`` and the query's
    document.  Per query that is the single range ``[max(doc_start[q], (q // block - w + 1) * block), q]``,
    which the attention kernel takes as a per-row lower bound.  Layers cycle long, short, short,
    short, ... with the last layer long; short = long // 2.  Returns a list of ``num_layers``
    ``WindowMask`` objects (two distinct ones) for ``CausalSelfAttention.forward(block_mask=...)``.
    """
    ids = input_seq.reshape(-1)
    T = ids.numel()
    torch._assert(T % block == 0, f"input_seq length {T} must be divisible by BLOCK_SIZE {block}")
    w_long = int(sliding_window_num_blocks)
    ds = doc_start_from_ids(ids, eos_token_id)
    qblk = torch.arange(T, device=ids.device, dtype=torch.int32) // block

    def one(w: int) -> WindowMask:
        lo_blk = torch.clamp_min(qblk - (max(w, 1) - 1), 0) * block
        return WindowMask(None, torch.maximum(ds, lo_blk).to(torch.int32).contiguous())

    long_m, short_m = one(w_long), one(w_long // 2)
    cycle = [long_m] + [short_m] * 3
    return (cycle * ((num_layers + 3) // 4))[:num_layers - 1] + [long_m]


def dense_mask_to_window(attn_mask: Tensor) -> WindowMask:
    """Converts a reference-style additive mask ``[..., T, T]`` to a ``WindowMask``.

    Raises if some row is not a single run of allowed keys ending at the query, or if the first
    allowed key moves backwards from one row to the next (the kernel chooses the key tiles of a
    block of queries from the block's first row).
    """
    m = attn_mask.reshape(-1, attn_mask.shape[-2], attn_mask.shape[-1])
    torch._assert(m.shape[0] == 1, "a dense attn_mask must broadcast over batch and heads")
    allowed = m[0] == 0
    T = allowed.shape[0]
    pos = torch.arange(T, device=allowed.device)
    first = torch.argmax(allowed.to(torch.int8), dim=1)
    count = allowed.sum(dim=1)
    band = (pos[None, :] >= first[:, None]) & (pos[None, :] <= pos[:, None])
    if not bool((count == pos - first + 1).all()) or not bool((allowed == band).all()):
        raise ValueError("attn_mask is not a causal band per row; only window/document masks are supported")
    if not bool((first[1:] >= first[:-1]).all()):
        raise ValueError("attn_mask's first allowed key decreases along the sequence; not supported")
    return WindowMask(None, first.to(torch.int32).contiguous())


def _marked_blocks(num: Tensor, indices: Tensor) -> Tensor:
    """Boolean ``[rows, cols]``: entry (i, j) set when j is among the first ``num[i]`` of ``indices[i]``."""
    rows, cols = indices.shape
    keep = torch.arange(cols, device=indices.device)[None, :] < num[:, None].long()
    dense = torch.zeros(rows, cols + 1, dtype=torch.bool, device=indices.device)
    dense[torch.arange(rows, device=indices.device)[:, None].expand(rows, cols),
          torch.where(keep, indices.long(), torch.full_like(indices, cols, dtype=torch.long))] = True
    return dense[:, :cols]


def block_mask_to_window(block_mask, pairs_per_pass: int = 256) -> WindowMask:
    """Converts a ``torch.nn.attention.flex_attention.BlockMask`` to a ``WindowMask``.

    The reference's training forward hands such an object to ``forward(block_mask=...)``
    (models/daisy/attention.py:156-171, built at models/daisy/daisy_core.py:209-221): per query
    block a list of *full* key blocks (every pair visible) and a list of *partial* ones (pairs
    filtered by ``mask_mod``).  The attention kernel takes one lower bound per query instead, so
    the set of visible keys of every row must be one run ``[lo(q), q]`` with ``lo`` non-decreasing
    -- which is what causal / sliding-window / document masks give.  The conversion evaluates
    ``mask_mod`` once on the partial blocks (as ``flex_attention`` itself does), derives ``lo``
    and verifies both conditions; anything else raises ``ValueError``.
    """
    qb_size, kb_size = block_mask.BLOCK_SIZE
    num_p, idx_p = block_mask.kv_num_blocks, block_mask.kv_indices
    torch._assert(num_p.dim() == 3 and num_p.shape[0] == 1 and num_p.shape[1] == 1,
                  "a BlockMask must have batch and head dimensions of 1 (one mask shared by all)")
    num_p, idx_p = num_p[0, 0], idx_p[0, 0]
    dev = idx_p.device
    nqb, nkb = idx_p.shape
    q_len, kv_len = block_mask.seq_lengths
    torch._assert(q_len == kv_len, "a BlockMask for self-attention must be square")
    T = q_len
    partial = _marked_blocks(num_p, idx_p)
    if block_mask.full_kv_num_blocks is not None:
        full = _marked_blocks(block_mask.full_kv_num_blocks[0, 0], block_mask.full_kv_indices[0, 0])
    else:
        full = torch.zeros_like(partial)
    mask_mod = block_mask.mask_mod
    big = T + kb_size
    q_of_block = torch.arange(nqb, device=dev)[:, None] * qb_size + torch.arange(qb_size, device=dev)[None, :]   # [nqb, qb]
    # full blocks: every key of the block is visible to every row of the query block
    kb_first = torch.arange(nkb, device=dev) * kb_size
    kb_last = torch.clamp_max(kb_first + kb_size, T) - 1
    first_full = torch.where(full, kb_first[None, :], big).min(dim=1).values                     # [nqb]
    last_full = torch.where(full, kb_last[None, :], -1).max(dim=1).values
    count_full = (full * (kb_last - kb_first + 1)[None, :]).sum(dim=1)
    lo = first_full[:, None].expand(nqb, qb_size).clone()
    hi = last_full[:, None].expand(nqb, qb_size).clone()
    count = count_full[:, None].expand(nqb, qb_size).clone()
    # partial blocks: mask_mod decides pair by pair
    pairs = torch.nonzero(partial & ~full)
    zero = torch.zeros((), dtype=torch.long, device=dev)
    for s in range(0, pairs.shape[0], pairs_per_pass):
        qi, kj = pairs[s:s + pairs_per_pass, 0], pairs[s:s + pairs_per_pass, 1]
        qs = (qi[:, None] * qb_size + torch.arange(qb_size, device=dev)[None, :])[:, :, None]     # [P, qb, 1]
        ks = (kj[:, None] * kb_size + torch.arange(kb_size, device=dev)[None, :])[:, None, :]     # [P, 1, kb]
        inside = (qs < T) & (ks < T)
        seen = mask_mod(zero, zero, torch.clamp_max(qs, T - 1), torch.clamp_max(ks, T - 1)) & inside
        row_lo = torch.where(seen, ks, big).amin(dim=2)                                           # [P, qb]
        row_hi = torch.where(seen, ks, -1).amax(dim=2)
        row_n = seen.sum(dim=2)
        rows_of = qi[:, None].expand_as(row_lo)
        lo.scatter_reduce_(0, rows_of, row_lo, "amin")
        hi.scatter_reduce_(0, rows_of, row_hi, "amax")
        count.index_add_(0, qi, row_n)
    lo, hi, count = lo.reshape(-1)[:T], hi.reshape(-1)[:T], count.reshape(-1)[:T]
    q = q_of_block.reshape(-1)[:T]
    if not bool(((hi == q) & (count == q - lo + 1)).all()):
        raise ValueError("block_mask does not describe one run of keys ending at each query; only causal "
                         "window / document masks are supported")
    if not bool((lo[1:] >= lo[:-1]).all()):
        raise ValueError("block_mask's first visible key decreases along the sequence; not supported")
    return WindowMask(None, lo.to(torch.int32).contiguous())


def _is_flex_block_mask(obj) -> bool:
    return all(hasattr(obj, a) for a in ("kv_num_blocks", "kv_indices", "mask_mod", "BLOCK_SIZE"))


MaskLike = Union[None, WindowMask, Tensor, "torch.nn.attention.flex_attention.BlockMask"]


class _ConvertedMasks:
    """Remembers the descriptors made from dense masks and BlockMask objects.

    The reference hands one mask object to every layer of a pass (daisy_core.py:251-262,338-345) and
    a conversion reads every entry of the mask and synchronises, so it is done once per object: the
    entries are keyed by the object's identity, hold it weakly and, for tensors, are dropped when the
    tensor was written to since (its version counter moved).
    """

    def __init__(self, limit: int = 16):
        self._entries: dict = {}
        self._limit = limit

    def get(self, obj, convert) -> WindowMask:
        key = id(obj)
        version = getattr(obj, "_version", 0)
        hit = self._entries.get(key)
        if hit is not None and hit[0]() is obj and hit[1] == version:
            return hit[2]
        converted = convert(obj)
        if len(self._entries) >= self._limit:
            self._entries = {k: e for k, e in self._entries.items() if e[0]() is not None}
            while len(self._entries) >= self._limit:
                self._entries.pop(next(iter(self._entries)))
        try:
            self._entries[key] = (weakref.ref(obj), version, converted)
        except TypeError:     # an object that cannot be referenced weakly is converted every time
            pass
        return converted


_converted_masks = _ConvertedMasks()


def _as_window_mask(attn_mask) -> WindowMask:
    if attn_mask is None:
        return WindowMask(None, None)
    if isinstance(attn_mask, WindowMask):
        return attn_mask
    if isinstance(attn_mask, Tensor):
        return _converted_masks.get(attn_mask, dense_mask_to_window)
    if _is_flex_block_mask(attn_mask):
        return _converted_masks.get(attn_mask, block_mask_to_window)
    raise TypeError(f"unsupported attn_mask type {type(attn_mask).__name__}")


def _apply_rope(x_BTHD: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    # Used for single-token tensors only; the prefill kernel rotates in registers.
    x1, x2 = x_BTHD.to(dtype=torch.float32).chunk(2, dim=-1)
    y1 = x1 * cos + x2 * sin
    y2 = x1 * (-sin) + x2 * cos
    return torch.cat((y1, y2), dim=-1).type_as(x_BTHD)


class Rotary(nn.Module):
    """Half-truncated RoPE tables (models/daisy/attention.py:26-70).

    The first ``dim // 4`` frequencies are ``(1/1024) ** linspace(0, 1, dim // 4)``,
    the remaining ``dim // 4`` are zero; ``dim < 4`` keeps all ``dim // 2``.  Tables
    are fp32 ``[max_seq_len, dim // 2]`` non-persistent buffers.
    """

    def __init__(self, dim: int, max_seq_len: int):
        super().__init__()
        half, keep = dim // 2, dim // 4
        base = 1024
        if keep == 0:
            angular_freq = (1 / base) ** torch.linspace(0, 1, steps=half, dtype=torch.float32)
        else:
            active = (1 / base) ** torch.linspace(0, 1, steps=keep, dtype=torch.float32)
            angular_freq = torch.cat([active, active.new_zeros(half - keep)])
        self.inv_freq = nn.Buffer(angular_freq, persistent=False)
        self._inv_freq_fp32 = angular_freq.clone()   # plain attribute: survives dtype casts of the module
        theta = torch.outer(torch.arange(max_seq_len, dtype=torch.float32), angular_freq)
        self.cos = nn.Buffer(theta.cos(), persistent=False)
        self.sin = nn.Buffer(theta.sin(), persistent=False)
        self._max_seq_len = int(max_seq_len)

    def _apply(self, fn, recurse=True):
        # Module-wide casts (model.bfloat16(), .half(), .to(dtype)) move the tables with the module
        # but must not narrow them: the kernels take fp32 tables, and bf16 angles lose the position.
        super()._apply(fn, recurse)
        for name in ("inv_freq", "cos", "sin"):
            buf = getattr(self, name)
            if buf.dtype != torch.float32:
                dev = buf.device
                if name == "inv_freq":
                    fresh = self._inv_freq_fp32.to(dev)
                else:
                    # rebuilt where the constructor built them, on the CPU: the GPU's cos / sin differ from the
                    # CPU's in the last bit, and the tables are to stay what the reference's constructor computes
                    theta = torch.outer(torch.arange(self._max_seq_len, dtype=torch.float32), self._inv_freq_fp32.cpu())
                    fresh = (theta.cos() if name == "cos" else theta.sin()).to(dev)
                setattr(self, name, nn.Buffer(fresh, persistent=False))
        return self

    def _get_cos_sin(self, L):
        torch._assert(L <= self.cos.shape[0], f"Rotary buffers too small {self.cos.shape[0]} < {L}")
        return self.cos.narrow(0, 0, L), self.sin.narrow(0, 0, L)

    def forward(self, x_BTHD: Tensor):
        cos, sin = self._get_cos_sin(x_BTHD.size(-3))
        return _apply_rope(x_BTHD, cos[None, :, None, :], sin[None, :, None, :])

    def step(self, x_BTHD: Tensor, pos: int):
        torch._assert(x_BTHD.size(1) == 1, "step() requires single position only")
        cos, sin = self._get_cos_sin(pos + 1)
        return _apply_rope(x_BTHD, cos[None, pos:pos + 1, None, :], sin[None, pos:pos + 1, None, :])


# Up to this many sequences, a decode step's two projections go through ``ops.linear_rows`` (the weights are read
# once by a kernel made for a few rows: 4.6 against 9.9 us for a 4608 x 1536 matrix and one row); beyond, the library GEMM.
STEP_ROWS_KERNEL_MAX = 4


def step_linear(x: Tensor, w: Tensor) -> Tensor:
    """``F.linear(x, w)`` for the activations of a decode step (models/daisy/attention.py:119-120, :201).
    The kernel has no backward: where autograd would record the product, the library op stays."""
    if (x.numel() <= STEP_ROWS_KERNEL_MAX * x.shape[-1] and ops.linear_rows_ok(x, w)
            and not (torch.is_grad_enabled() and (x.requires_grad or w.requires_grad))):
        return ops.linear_rows(x, w)
    return F.linear(x, w)


class CausalSelfAttention(nn.Module):
    """Merged-QKVO sliding-window causal self-attention (models/daisy/attention.py:73-202)."""

    # step() takes a KVCache layer handle (RingContext) in place of chronological k_ctx / v_ctx.
    accepts_ring_context = True

    def __init__(self, dim: int, num_heads: int, head_dim, receives_ve: bool = False,
                 layer_idx: Optional[int] = None, max_seq_len: int = 131072):
        super().__init__()
        torch._assert(dim % num_heads == 0, "dim must be divisible by num_heads")
        self.num_heads = num_heads
        self.head_dim: int = head_dim
        self.m_dim = dim
        self.qkvo_w = nn.Parameter(init_linear(torch.empty(4, dim, dim)).bfloat16())
        if os.getenv("DISABLE_O_ZERO_INIT", "") != "1":
            self.qkvo_w.detach()[3].zero_()
        self.rotary = Rotary(head_dim, max_seq_len)
        self.attn_scale = 0.12
        self.last_q = None
        self.last_k = None
        self.receives_ve = receives_ve
        if receives_ve:
            # Gate logits per layer as in the reference (attention.py:94-106).
            ve_init_logits = {0: 0.3228, 1: 0.0, 2: -1.5163, 21: -2.4423, 22: -2.9444, 23: 10.0}
            init_val = ve_init_logits.get(layer_idx, 0.0) if layer_idx is not None else 0.0
            self.g_ve = nn.Parameter(torch.tensor(init_val))
        else:
            self.g_ve = None
        self.debug_logging = False
        # Norm + RoPE + ve mix in one streaming kernel ahead of attention (bf16 weights only);
        # False keeps norm / mix in PyTorch and rotates inside the attention call.
        self.fused_prep = True

    def reset_history(self):
        self.last_q = None
        self.last_k = None

    # -- shared pieces -------------------------------------------------------
    def _project_qkv(self, x: Tensor):
        """QKV projection + RMS norm of q, k and v (no RoPE); ``[B, T, H, D]`` views."""
        B, T = x.size(0), x.size(1)
        x = x.to(self.qkvo_w.dtype)
        qkv = step_linear(x, self.qkvo_w[:3].flatten(end_dim=1)).view(B, T, 3 * self.num_heads, self.head_dim)
        q, k, v = qkv.chunk(3, dim=-2)
        return norm(q), norm(k), norm(v)

    def _mix_ve(self, v: Tensor, ve: Optional[Tensor]) -> Tensor:
        if not self.receives_ve:
            return v
        torch._assert(ve is not None, "ve must be provided when receives_ve=True")
        g_x = torch.sigmoid(self.g_ve).to(v.dtype)
        return g_x * v + (1.0 - g_x) * ve.view_as(v).to(v.dtype)

    def _kernel_dtype(self, t: Tensor) -> Tensor:
        # The kernels compute on bf16 operands; fp32 parameters (as some tests
        # use) are rounded here and the result is widened again by the caller.
        return t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)

    def _fused_prep_ok(self) -> bool:
        # The one-pass norm + RoPE + ve-mix kernel works on bf16 rows of 64 or 128 channels.
        return self.fused_prep and self.qkvo_w.dtype == torch.bfloat16 and self.head_dim in (64, 128)

    def _project_qkv_fused(self, x: Tensor, ve: Optional[Tensor], pos0: int, k_out=None, v_out=None):
        """QKV projection, then norm + RoPE (rows ``pos0 + t``) + ve mix in one kernel; ``[B, T, H, D]``.
        ``k_out`` / ``v_out``: strided ``[B, T, H, D]`` views that receive k and v (e.g. slots of a ring cache)."""
        B, T = x.size(0), x.size(1)
        x = x.to(self.qkvo_w.dtype)
        qkv = step_linear(x, self.qkvo_w[:3].flatten(end_dim=1)).view(B, T, 3 * self.num_heads, self.head_dim)
        q, k, v = qkv.chunk(3, dim=-2)
        gate = None
        if self.receives_ve:
            torch._assert(ve is not None, "ve must be provided when receives_ve=True")
            ve = ve.to(torch.bfloat16).view(B, T, self.num_heads, self.head_dim)
            gate = torch.sigmoid(self.g_ve.detach()).to(torch.bfloat16).float().reshape(1)
        else:
            ve = None
        if isinstance(pos0, Tensor):
            cos, sin = self.rotary.cos, self.rotary.sin   # position known on the device only: whole tables
        else:
            cos, sin = self.rotary._get_cos_sin(pos0 + T)
        return ops.qkv_prep(q, k, v, eps=NORM_EPS_BF16, cos=cos, sin=sin, pos0=pos0, ve=ve, gate=gate,
                            k_out=k_out, v_out=v_out)

    def _attend(self, x: Tensor, ve: Optional[Tensor], attn_mask, kv_out=None, want_q: bool = False):
        """Returns ``y [B, T, dim]`` and q (rotated), k (rotated), v as ``[B, T, H, D]``.  Where the kernels
        rotate q themselves, the rotated q is computed for the caller only when ``want_q`` asks for it
        (``prefill(debug=True)``), and is ``None`` otherwise."""
        B, T = x.size(0), x.size(1)
        mask = _as_window_mask(attn_mask)
        if mask.doc_start is not None and mask.doc_start.device != x.device:    # e.g. converted from a mask built on the CPU
            mask = WindowMask(mask.window, mask.doc_start.to(x.device), mask.kv_out)
        dest = kv_out if kv_out is not None else mask.kv_out
        if self._fused_prep_ok():
            q, k_rot, v = self._project_qkv_fused(x, ve, 0, *(dest or (None, None)))
            o, _ = ops.prefill_attention(q, k_rot, v, window=mask.window, scale=self.attn_scale, doc_start=mask.doc_start)
            y = F.linear(o.view(B, T, self.m_dim), self.qkvo_w[3])
            return y, q, k_rot, v
        torch._assert(dest is None, "writing keys and values to a destination needs the fused pre-attention kernel")
        q, k, v = self._project_qkv(x)
        dtype = q.dtype
        v = self._mix_ve(v, ve)
        cos, sin = self.rotary._get_cos_sin(T)
        if dtype == torch.float32:
            # fp32 parameters (the reference's unit tests build the module so): fp32 tensors and fp32
            # arithmetic through the attention too, nothing is rounded to bf16 on the way.
            q_rot = _apply_rope(q, cos[None, :, None, :], sin[None, :, None, :]) if want_q else None
            o, k_rot = ops.prefill_attention_f32(q, k, v, window=mask.window, scale=self.attn_scale, cos=cos, sin=sin,
                                                 doc_start=mask.doc_start)
            y = F.linear(o.view(B, T, self.m_dim), self.qkvo_w[3])
            return y, q_rot, k_rot, v
        o, k_rot = ops.prefill_attention(
            self._kernel_dtype(q), self._kernel_dtype(k), self._kernel_dtype(v),
            window=mask.window, scale=self.attn_scale, cos=cos, sin=sin, doc_start=mask.doc_start)
        y = o.view(B, T, self.m_dim).to(dtype)
        y = F.linear(y, self.qkvo_w[3])
        q_rot = _apply_rope(q, cos[None, :, None, :], sin[None, :, None, :]) if want_q else None
        return y, q_rot, k_rot.to(dtype), v

    # -- reference interface -----------------------------------------------
    def forward(self, x: Tensor, ve: Optional[Tensor], block_mask=None, attn_mask: MaskLike = None):
        """``block_mask``: a ``WindowMask``, or the ``flex_attention`` ``BlockMask`` the reference's
        training forward builds (models/daisy/daisy_core.py:209-221), converted once per object to
        per-row bounds (``block_mask_to_window``).  Forward only: the kernels have no backward."""
        y, _, _, _ = self._attend(x, ve, block_mask if block_mask is not None else attn_mask)
        return y

    def forward_sdpa(self, x: Tensor, ve: Optional[Tensor], attn_mask: MaskLike = None):
        return self.forward(x, ve, attn_mask=attn_mask)

    def prefill(self, x: Tensor, ve: Optional[Tensor], attn_mask: MaskLike = None, debug: bool = False, kv_out=None):
        """Returns ``y [B, T, dim]``, ``k [B, H, T, D]`` (normed + rotated), ``v [B, H, T, D]``.

        ``kv_out``: ``(k, v)`` destination views ``[B, T, H, D]`` (see ``WindowMask.kv_out``, which is
        the way through a ``Block`` that passes only the reference's arguments on).
        ``debug`` keeps the rotated q and k as ``last_q`` / ``last_k`` like the reference
        (attention.py:176-178), as copies when they alias a destination that later steps overwrite."""
        y, q, k, v = self._attend(x, ve, attn_mask, kv_out, want_q=debug)
        if debug:
            aliased = kv_out is not None or getattr(_as_window_mask(attn_mask), "kv_out", None) is not None
            self.last_q = q
            self.last_k = k.clone() if aliased else k
        return y, k.transpose(1, 2), v.transpose(1, 2)

    def step(self, x, k_ctx: Union[Tensor, RingContext], v_ctx: Union[Tensor, RingContext], pos: Union[int, Tensor],
             ve: Optional[Tensor], window: Optional[int]):
        """One token: returns ``y [B, 1, dim]``, ``k [B, 1, H, D]``, ``v [B, 1, H, D]``.

        ``k_ctx``/``v_ctx`` are either the chronological cached rows
        ``[B, n, H, D]`` (the reference's calling convention) or the
        ``RingContext`` of a ``KVCache`` layer, in which case the kernel streams
        the ring in place and appends the new row itself.

        ``pos`` may be a one-element int32 device tensor (with a ``RingContext`` only): nothing on
        the host then depends on the position, so the step can be recorded in a HIP graph and
        replayed while the tensor counts up.
        """
        B = x.size(0)
        torch._assert(x.size(1) == 1, "step() requires single position only")
        fused = self._fused_prep_ok()
        ring = k_ctx if isinstance(k_ctx, RingContext) else None
        # the one-launch step streams a bf16 ring, or an fp16 one (the reference generator's default)
        in_ring = fused and ring is not None and ring.k.dtype in (torch.bfloat16, torch.float16) and window == ring.W
        if isinstance(pos, Tensor):
            if not in_ring:
                raise ValueError("a device-side position needs the fused kernels (bf16 weights, head dim 64 or 128) "
                                 "and the RingContext of a bf16 or fp16 KVCache whose size equals the window")
            return self._step_in_ring(x, ring, pos, ve)
        if in_ring and pos == ring.t:
            return self._step_in_ring(x, ring, pos, ve)
        if fused:
            # q and k come back rotated: the decode kernel is told not to rotate again.
            q, k, v = self._project_qkv_fused(x, ve, pos)
            dtype = q.dtype
            cos_row = sin_row = None
        else:
            q, k, v = self._project_qkv(x)
            dtype = q.dtype
            v = self._mix_ve(v, ve)
            cos, sin = self.rotary._get_cos_sin(pos + 1)
            cos_row, sin_row = cos[pos], sin[pos]
        if dtype == torch.float32:
            return self._step_f32(q, k, v, k_ctx, v_ctx, pos, window, cos_row, sin_row)
        qk, kk, vk = (self._kernel_dtype(t)[:, 0] for t in (q, k, v))  # [B, H, D]

        if ring is not None and (window != ring.W or ring.k.dtype != torch.bfloat16 or pos != ring.t):
            # Not the layout the in-place path streams; use the chronological rows.
            k_ctx, v_ctx = ring.cache.view(ring.layer)
            ring = None
        if ring is not None:
            W, t = ring.W, ring.t
            slot = t % W
            o = ops.decode_attention(qk, kk, vk, ring.k, ring.v, n_rows=min(t + 1, W), new_idx=slot,
                                     write_back=True, scale=self.attn_scale, cos_row=cos_row, sin_row=sin_row)
            ring.mark_written()
            k_new = ring.k[:, :, slot, :].unsqueeze(1)
            v_new = ring.v[:, :, slot, :].unsqueeze(1)
        else:
            n = k_ctx.size(1)
            r = n if window is None else min(n, max(window - 1, 0))
            if fused:
                k_new, v_new, q_rot = k, v, q
            else:
                k_new = _apply_rope(self._kernel_dtype(k), cos_row[None, None, None, :], sin_row[None, None, None, :])
                v_new = self._kernel_dtype(v)
                q_rot = _apply_rope(self._kernel_dtype(q), cos_row[None, None, None, :], sin_row[None, None, None, :])
            if r > 0:
                kc = self._kernel_dtype(k_ctx)[:, n - r:n].transpose(1, 2)  # [B, H, r, D] view
                vc = self._kernel_dtype(v_ctx)[:, n - r:n].transpose(1, 2)
            else:
                kc = vc = None
            o = ops.decode_attention(q_rot[:, 0], k_new[:, 0], v_new[:, 0], kc, vc, n_rows=r + 1, new_idx=r,
                                     write_back=False, scale=self.attn_scale)
            k_new, v_new = k_new.to(dtype), v_new.to(dtype)
        y = o.reshape(B, 1, self.m_dim).to(dtype)
        y = step_linear(y, self.qkvo_w[3])
        return y, k_new, v_new

    def _step_f32(self, q, k, v, k_ctx, v_ctx, pos, window, cos_row, sin_row):
        """The step of a module with fp32 parameters: fp32 tensors and arithmetic throughout
        (``ops.decode_attention_f32``); the cached rows are taken as fp32 whatever the cache holds."""
        B = q.size(0)
        if isinstance(k_ctx, RingContext):
            k_ctx, v_ctx = k_ctx.cache.view(k_ctx.layer)
        n = k_ctx.size(1)
        r = n if window is None else min(n, max(window - 1, 0))
        kc = vc = None
        if r > 0:
            kc = k_ctx[:, n - r:n].float().transpose(1, 2)      # [B, H, r, D] view
            vc = v_ctx[:, n - r:n].float().transpose(1, 2)
        o = ops.decode_attention_f32(q[:, 0], k[:, 0], v[:, 0], kc, vc, n_rows=r + 1, new_idx=r, scale=self.attn_scale,
                                     cos_row=cos_row.contiguous(), sin_row=sin_row.contiguous())
        y = F.linear(o.reshape(B, 1, self.m_dim), self.qkvo_w[3])
        k_new = _apply_rope(k, cos_row[None, None, None, :], sin_row[None, None, None, :])
        return y, k_new, v

    def _step_in_ring(self, x, ring: RingContext, pos: Union[int, Tensor], ve: Optional[Tensor]):
        """The step as two projections around one kernel: norm, RoPE, value-embedding mix, the new
        rows' way into slot ``pos % W`` and the attention over the ring all happen in
        ``ops.attn_step``.  Returns the new rows as views of the ring, or ``None, None`` when only
        the device knows the position."""
        B, H, D = x.size(0), self.num_heads, self.head_dim
        x = x.to(self.qkvo_w.dtype)
        ve_rows = gate = None
        if self.receives_ve:
            torch._assert(ve is not None, "ve must be provided when receives_ve=True")
            ve_rows = ve.to(torch.bfloat16).view(B, H, D)
            gate = torch.sigmoid(self.g_ve.detach()).to(torch.bfloat16).float().reshape(1)
        status = ring.status if isinstance(pos, Tensor) else None
        w_qkv, w_out = self.qkvo_w[:3].flatten(end_dim=1), self.qkvo_w[3]
        if (B <= STEP_ROWS_KERNEL_MAX and x.is_contiguous() and H * D == self.m_dim and ops.linear_rows_ok(x, w_qkv)
                and not (torch.is_grad_enabled() and (x.requires_grad or w_qkv.requires_grad))):
            # a few sequences: both projections and the attention step go out in one call
            y = ops.attn_layer_step(x, w_qkv, w_out, ring.k, ring.v, pos, cos=self.rotary.cos, sin=self.rotary.sin,
                                    eps=NORM_EPS_BF16, ve=ve_rows, gate=gate, scale=self.attn_scale, status=status)
            ring.mark_written()
        else:
            qkv = step_linear(x, w_qkv).view(B, 3 * H, D)
            o = ops.attn_step(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], ring.k, ring.v, pos,
                              cos=self.rotary.cos, sin=self.rotary.sin, eps=NORM_EPS_BF16, ve=ve_rows, gate=gate,
                              scale=self.attn_scale, status=status)
            ring.mark_written()
            y = step_linear(o.reshape(B, 1, self.m_dim), w_out)
        if isinstance(pos, Tensor):
            return y, None, None
        slot = pos % ring.W
        k_new, v_new = ring.k[:, :, slot, :].unsqueeze(1), ring.v[:, :, slot, :].unsqueeze(1)
        if k_new.dtype != y.dtype:      # an fp16 ring: the rows go back in the model's dtype, as the reference's do
            k_new, v_new = k_new.to(y.dtype), v_new.to(y.dtype)
        return y, k_new, v_new
