"""Kimi Delta Attention entry points with the names the reference calls.

``chunk_kda`` stands in for ``fla.ops.kda.chunk_kda`` as called at
models/daisy/attention_kimi.py:133-134 and ``fused_kda_gate`` for
models/daisy/fla_custom_ops.py:190-200 (forward only).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from . import ops


def _per_sequence(kernel, q, k, v, g, beta, initial_state, output_final_state, cu_seqlens, **kw):
    """Variable-length packing: ``B == 1`` and sequence i occupies positions
    ``[cu_seqlens[i], cu_seqlens[i+1])`` of the T axis; states are ``[N, H, Dk, Dv]``.  Every
    sequence is one kernel call on its slice (the boundaries are read on the host, as the
    chunk index tables of the reference's kernels are)."""
    torch._assert(q.size(0) == 1, "cu_seqlens needs batch size 1 (sequences packed along T)")
    bounds = [int(x) for x in cu_seqlens.tolist()]
    n_seq = len(bounds) - 1
    torch._assert(n_seq >= 1 and bounds[0] == 0 and bounds[-1] == q.size(1), "cu_seqlens must run from 0 to T")
    if initial_state is not None:
        torch._assert(initial_state.size(0) == n_seq, "initial_state needs one state per sequence")
    outs, finals = [], []
    for i in range(n_seq):
        s, e = bounds[i], bounds[i + 1]
        torch._assert(e >= s, "cu_seqlens must not decrease")
        s0 = initial_state[i:i + 1] if initial_state is not None else None
        if e == s:   # an empty sequence leaves its state as it was
            if output_final_state:
                finals.append(s0.clone() if s0 is not None else
                              torch.zeros(1, q.size(2), q.size(3), v.size(3), device=q.device, dtype=torch.float32))
            continue
        o_i, f_i = kernel(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e], initial_state=s0,
                          output_final_state=output_final_state, **kw)
        outs.append(o_i)
        if output_final_state:
            finals.append(f_i)
    o = torch.cat(outs, dim=1) if outs else v.new_zeros(v.shape)
    return o, (torch.cat(finals, dim=0) if output_final_state else None)


def chunk_kda(q: Tensor, k: Tensor, v: Tensor, g: Tensor, beta: Tensor, scale: Optional[float] = None,
              initial_state: Optional[Tensor] = None, output_final_state: bool = False,
              use_qk_l2norm_in_kernel: bool = False, cu_seqlens: Optional[Tensor] = None):
    """Chunked gated delta rule with per-channel decay.

    ``q, k, g [B, T, H, Dk]``, ``v [B, T, H, Dv]``, ``beta [B, T, H]``; returns
    ``(o [B, T, H, Dv], final_state [B, H, Dk, Dv] or None)``.  ``scale`` defaults
    to ``Dk ** -0.5``.  With ``cu_seqlens [N + 1]`` the batch is 1 and holds N sequences packed
    along T, each with its own state (``initial_state`` / ``final_state [N, H, Dk, Dv]``).
    """
    if cu_seqlens is not None:
        return _per_sequence(chunk_kda, q, k, v, g, beta, initial_state, output_final_state, cu_seqlens,
                             scale=scale, use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel)
    bf = lambda t: t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)
    o, final = ops.kda_chunk_fwd(bf(q), bf(k), bf(v), g, beta, scale=scale, initial_state=initial_state,
                                 output_final_state=output_final_state,
                                 use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel)
    return o.to(v.dtype), final


def fused_recurrent_kda(q: Tensor, k: Tensor, v: Tensor, g: Tensor, beta: Tensor, scale: Optional[float] = None,
                        initial_state: Optional[Tensor] = None, output_final_state: bool = False,
                        use_qk_l2norm_in_kernel: bool = False, cu_seqlens: Optional[Tensor] = None,
                        inplace_state: bool = False):
    """Same arguments and results as ``chunk_kda``, evaluated token by token with the state in
    registers: the mode for single-token decode steps (``T == 1``, state carried by the caller)
    and short prompts.  ``models/daisy/attention_kimi.py:70,144`` names this mode
    (``'fused_recurrent'``) without supporting it.
    """
    if cu_seqlens is not None:
        torch._assert(not inplace_state, "inplace_state does not combine with cu_seqlens")
        return _per_sequence(fused_recurrent_kda, q, k, v, g, beta, initial_state, output_final_state, cu_seqlens,
                             scale=scale, use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel)
    bf = lambda t: t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)
    o, final = ops.kda_recurrent_fwd(bf(q), bf(k), bf(v), g, beta, scale=scale, initial_state=initial_state,
                                     output_final_state=output_final_state or inplace_state,
                                     use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, inplace_state=inplace_state)
    return o.to(v.dtype), (final if (output_final_state or inplace_state) else None)


def fused_kda_gate(g: Tensor, A_log: Tensor, head_k_dim: int, g_bias: Optional[Tensor] = None,
                   b: Optional[Tensor] = None, beta: float = 1.0, threshold: float = 20.0):
    """``-exp(A_log) * softplus(g + bias)`` reshaped to ``[..., H, Dk]``; with ``b`` also ``sigmoid(b)``."""
    y = ops.kda_gate_fwd(g, A_log, head_k_dim, g_bias, beta, threshold)
    return y if b is None else (y, torch.sigmoid(b.to(dtype=g.dtype)))
