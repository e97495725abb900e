"""fp32 restatement of the reference's sliding-window causal self-attention.

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.
"""
from __future__ import annotations

from typing import Optional

import torch

ATTN_SCALE = 0.12  # models/daisy/attention.py:88


def rope_tables(head_dim: int, max_seq_len: int, base: float = 1024.0, half_truncate: bool = True):
    """cos/sin tables ``[max_seq_len, head_dim // 2]`` in fp32.

    Follows models/daisy/attention.py:27-49: the first ``head_dim // 4``
    frequencies are ``(1/base) ** linspace(0, 1, head_dim // 4)`` and the rest
    are zero ("half-truncated" RoPE); for ``head_dim < 4`` all ``head_dim // 2``
    frequencies are active.  ``half_truncate=False`` gives the plain table with
    ``head_dim // 2`` active frequencies (used by the benchmark configs that ask
    for an ordinary base-10000 table).
    """
    half = head_dim // 2
    keep = head_dim // 4
    if keep == 0 or not half_truncate:
        freq = (1.0 / base) ** torch.linspace(0, 1, steps=half, dtype=torch.float32)
    else:
        active = (1.0 / base) ** torch.linspace(0, 1, steps=keep, dtype=torch.float32)
        freq = torch.cat([active, active.new_zeros(half - keep)])
    t = torch.arange(max_seq_len, dtype=torch.float32)
    theta = t[:, None] * freq[None, :]
    return theta.cos(), theta.sin()


def apply_rope(x_BTHD: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate pairs (i, i + D/2): y1 = x1*cos + x2*sin, y2 = -x1*sin + x2*cos.

    models/daisy/attention.py:16-20.  ``cos``/``sin`` are ``[T, D/2]`` rows for
    the T positions of ``x`` (already sliced to the positions wanted).  Math in
    fp32, result cast back to the input dtype.
    """
    x = x_BTHD.to(torch.float32)
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c = cos[None, :, None, :]
    s = sin[None, :, None, :]
    y1 = x1 * c + x2 * s
    y2 = -x1 * s + x2 * c
    return torch.cat((y1, y2), dim=-1).to(x_BTHD.dtype)


def rms_norm(x: torch.Tensor) -> torch.Tensor:
    """Weightless RMS norm over the last dim, as ``F.rms_norm(x, (D,))`` with ``eps=None``.

    models/daisy/functional.py:6-7.  With ``eps=None`` the library (torch 2.10)
    uses the machine epsilon of its ACCUMULATION type -- fp32 for bf16, fp16 and
    fp32 inputs -- not ``finfo(x.dtype).eps``; the pin test compares against the
    library bit for bit.
    """
    acc = torch.float64 if x.dtype == torch.float64 else torch.float32
    eps = torch.finfo(acc).eps
    xf = x.to(acc)
    y = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return y.to(x.dtype)


def build_attn_mask(input_seq: torch.Tensor, window_size: int, eos_token_id: int) -> torch.Tensor:
    """Additive fp32 mask ``[1, 1, T, T]``: -inf where k > q, q - k >= window, or
    the two positions are in different documents; documents are numbered by
    ``cumsum(ids == eos)`` so an EOS token starts the document it belongs to.

    models/daisy/daisy_core.py:53-69.
    """
    ids = input_seq.reshape(-1)
    T = ids.numel()
    pos = torch.arange(T)
    d = pos[:, None] - pos[None, :]
    docs = (ids == eos_token_id).to(torch.int64).cumsum(0)
    m = torch.zeros(T, T, dtype=torch.float32)
    m[d < 0] = float("-inf")
    m[d >= window_size] = float("-inf")
    m[docs[:, None] != docs[None, :]] = float("-inf")
    return m[None, None]


def doc_start_from_ids(input_seq: torch.Tensor, eos_token_id: int) -> torch.Tensor:
    """int32 ``[T]``: index of the first token of the document holding each position.

    With ``docs = cumsum(ids == eos)`` (models/daisy/daisy_core.py:60) a position
    belongs to the document started by the latest EOS at or before it, so the
    document mask ``docs[q] == docs[k]`` for ``k <= q`` is ``k >= doc_start[q]``.
    """
    ids = input_seq.reshape(-1)
    T = ids.numel()
    out = torch.zeros(T, dtype=torch.int32)
    start = 0
    for i in range(T):
        if int(ids[i]) == eos_token_id:
            start = i
        out[i] = start
    return out


def block_mask_dense(input_seq: torch.Tensor, window_blocks: int, eos_token_id: int, block: int = 128) -> torch.Tensor:
    """Boolean ``[T, T]`` visibility of one training-time block mask.

    models/daisy/daisy_core.py:182-221 (``create_blockmasks`` / ``build_bm``), restated block by
    block with the semantics of ``BlockMask.from_kv_blocks``: per query block the key blocks that
    touch it causally and by document are split into *full* ones (strictly earlier, every row of
    both blocks in one document) and *partial* ones; both lists are ordered from the most recent
    block backwards; the first ``min(n_full, w - 1)`` full blocks are visible everywhere, the first
    ``min(n_partial, max(w - n_full, 1))`` partial blocks where ``q >= k`` and ``docs[q] == docs[k]``.
    """
    ids = input_seq.reshape(-1)
    T = ids.numel()
    assert T % block == 0
    nb = T // block
    docs = torch.cumsum((ids == eos_token_id).to(torch.int64), 0)
    lo = docs.view(nb, block)[:, 0]
    hi = docs.view(nb, block)[:, -1]
    pos = torch.arange(T)
    allowed = torch.zeros(T, T, dtype=torch.bool)
    for i in range(nb):
        full, partial = [], []
        for j in range(i, -1, -1):                       # most recent first
            any_ = (i >= j) and bool(lo[i] <= hi[j]) and bool(hi[i] >= lo[j])
            all_ = (i > j) and bool(lo[i] == hi[j]) and bool(hi[i] == lo[j])
            if any_ and all_:
                full.append(j)
            elif any_:
                partial.append(j)
        n_full = len(full)
        keep_partial = partial[:min(len(partial), max(window_blocks - n_full, 1))]
        keep_full = full[:min(n_full, max(window_blocks - 1, 0))]
        qs = pos[i * block:(i + 1) * block]
        for j in keep_full:
            allowed[i * block:(i + 1) * block, j * block:(j + 1) * block] = True
        for j in keep_partial:
            ks = pos[j * block:(j + 1) * block]
            m = (qs[:, None] >= ks[None, :]) & (docs[qs][:, None] == docs[ks][None, :])
            allowed[i * block:(i + 1) * block, j * block:(j + 1) * block] = m
    return allowed


def block_mask_cycle(num_layers: int, window_blocks: int):
    """Per-layer window (in blocks): long, short, short, short, ... and long for the last layer
    (models/daisy/daisy_core.py:224-229); short = long // 2."""
    cycle = [window_blocks] + [window_blocks // 2] * 3
    return (cycle * ((num_layers + 3) // 4))[:num_layers - 1] + [window_blocks]


def window_mask(T: int, window: Optional[int], doc_start: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Same mask as ``build_attn_mask`` expressed through (window, doc_start)."""
    pos = torch.arange(T)
    d = pos[:, None] - pos[None, :]
    m = torch.zeros(T, T, dtype=torch.float32)
    m[d < 0] = float("-inf")
    if window is not None and window > 0:
        m[d >= window] = float("-inf")
    if doc_start is not None:
        m[pos[None, :] < doc_start.to(torch.int64)[:, None]] = float("-inf")
    return m[None, None]


def sdpa(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor], scale: float) -> torch.Tensor:
    """softmax(scale * q k^T + mask) v in fp32; inputs ``[B, H, Tq, D]`` / ``[B, H, Tk, D]``.

    The arithmetic the reference gets from ``F.scaled_dot_product_attention``
    (models/daisy/attention.py:145,147,199).
    """
    qf, kf, vf = q.float(), k.float(), v.float()
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    if mask is not None:
        s = s + mask
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, vf)


def windowed_attention(q, k, v, window: Optional[int], scale: float = ATTN_SCALE,
                       doc_start: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Dense masked attention, ``[B, H, T, D]`` in, fp32 ``[B, H, T, D]`` out."""
    T = q.shape[2]
    return sdpa(q, k, v, window_mask(T, window, doc_start), scale)


def windowed_attention_blockwise(q, k, v, window: Optional[int], scale: float = ATTN_SCALE,
                                 doc_start: Optional[torch.Tensor] = None, block: int = 512,
                                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Same result as ``windowed_attention`` without a T x T mask.

    Processes query rows in blocks and gathers only the keys a block can see,
    so T = 65536 is affordable.  ``rows`` (1-D int64) restricts the computation
    to those query positions (output ``[B, H, len(rows), D]``).
    """
    B, H, T, D = q.shape
    qf, kf, vf = q.float(), k.float(), v.float()
    if rows is None:
        rows = torch.arange(T)
    out = torch.empty(B, H, rows.numel(), D, dtype=torch.float32)
    W = T if (window is None or window <= 0) else window
    for i0 in range(0, rows.numel(), block):
        r = rows[i0:i0 + block]
        lo = int(max(0, int(r.min()) - W + 1))
        hi = int(r.max()) + 1
        kk = torch.arange(lo, hi)
        d = r[:, None] - kk[None, :]
        m = torch.zeros(r.numel(), kk.numel(), dtype=torch.float32)
        m[d < 0] = float("-inf")
        m[d >= W] = float("-inf")
        if doc_start is not None:
            m[kk[None, :] < doc_start.to(torch.int64)[r][:, None]] = float("-inf")
        s = torch.matmul(qf[:, :, r], kf[:, :, lo:hi].transpose(-1, -2)) * scale + m
        out[:, :, i0:i0 + r.numel()] = torch.matmul(torch.softmax(s, dim=-1), vf[:, :, lo:hi])
    return out


def calc_qkv(x: torch.Tensor, qkvo_w: torch.Tensor, num_heads: int, head_dim: int,
             cos: torch.Tensor, sin: torch.Tensor, pos: Optional[int] = None):
    """Merged QKV projection, RMS norm of q, k AND v, RoPE on q and k.

    models/daisy/attention.py:116-127.  Returns q, k, v as ``[B, T, H, D]`` in the
    weight dtype.  ``pos`` selects one table row (decode); otherwise rows 0..T-1.
    """
    B, T = x.shape[0], x.shape[1]
    x = x.to(qkvo_w.dtype)
    w = qkvo_w[:3].flatten(end_dim=1)
    qkv = torch.nn.functional.linear(x, w).view(B, T, 3 * num_heads, head_dim)
    q, k, v = qkv.chunk(3, dim=-2)
    q, k, v = rms_norm(q), rms_norm(k), rms_norm(v)
    if pos is not None:
        c, s = cos[pos:pos + 1], sin[pos:pos + 1]
    else:
        c, s = cos[:T], sin[:T]
    return apply_rope(q, c, s), apply_rope(k, c, s), v


def _mix_ve(v, ve, g_ve):
    # models/daisy/attention.py:132-135,186-190
    if g_ve is None:
        return v
    g = torch.sigmoid(torch.as_tensor(g_ve, dtype=torch.float32)).to(v.dtype)
    return g * v + (1.0 - g) * ve.view_as(v).to(v.dtype)


def attn_prefill(x, qkvo_w, num_heads, head_dim, cos, sin, window: Optional[int],
                 doc_start: Optional[torch.Tensor] = None, ve=None, g_ve=None, scale: float = ATTN_SCALE):
    """``CausalSelfAttention.prefill`` (models/daisy/attention.py:141-150,173-179).

    Returns ``y [B, T, dim]`` (weight dtype), ``k [B, H, T, D]``, ``v [B, H, T, D]``
    where k is post-norm post-RoPE and v is post-norm post-ve-mix.  The softmax
    and both contractions run in fp32 whatever the weight dtype.
    """
    B, T = x.shape[0], x.shape[1]
    q, k, v = calc_qkv(x, qkvo_w, num_heads, head_dim, cos, sin)
    v = _mix_ve(v, ve, g_ve)
    q_, k_, v_ = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    o = windowed_attention(q_, k_, v_, window, scale, doc_start)
    y = o.transpose(1, 2).contiguous().view(B, T, num_heads * head_dim).to(qkvo_w.dtype)
    y = torch.nn.functional.linear(y, qkvo_w[3])
    return y, k_, v_


def attn_step(x, k_ctx, v_ctx, pos: int, qkvo_w, num_heads, head_dim, cos, sin,
              window: Optional[int], ve=None, g_ve=None, scale: float = ATTN_SCALE):
    """``CausalSelfAttention.step`` (models/daisy/attention.py:181-202).

    ``k_ctx``/``v_ctx`` are the chronological cached rows ``[B, n, H, D]``; the
    new token attends the last ``min(n, window - 1)`` of them plus itself.
    Returns ``y [B, 1, dim]``, ``k [B, 1, H, D]``, ``v [B, 1, H, D]``.
    """
    B = x.shape[0]
    q, k, v = calc_qkv(x, qkvo_w, num_heads, head_dim, cos, sin, pos)
    v = _mix_ve(v, ve, g_ve)
    n = k_ctx.shape[1]
    r = n if window is None else min(n, max(window - 1, 0))
    k_ = torch.cat([k_ctx[:, n - r:n].to(k.dtype), k], 1).transpose(1, 2)
    v_ = torch.cat([v_ctx[:, n - r:n].to(v.dtype), v], 1).transpose(1, 2)
    o = sdpa(q.transpose(1, 2), k_, v_, None, scale)
    y = o.transpose(1, 2).contiguous().view(B, 1, num_heads * head_dim).to(qkvo_w.dtype)
    y = torch.nn.functional.linear(y, qkvo_w[3])
    return y, k, v


def prefill_flops(B: int, T: int, H: int, D: int, window: Optional[int]) -> float:
    """Algorithmic flops of windowed causal attention: 4*D*B*H*pairs."""
    if window is None or window <= 0 or window >= T:
        pairs = T * (T + 1) // 2
    else:
        pairs = window * (window + 1) // 2 + (T - window) * window
    return 4.0 * D * B * H * pairs


def decode_bytes(B: int, H: int, D: int, rows: int, elt: int = 2) -> int:
    """Algorithmic K+V bytes streamed by one decode step."""
    return B * H * rows * D * 2 * elt

