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


def chunk_kda(q: Tensor, k: Tensor, v: Tensor, g: Tensor, beta: Tensor, scale: Optional[float] = None,
              initial_state: Optional[Tensor] = None, output_final_state: bool = False,
              use_qk_l2norm_in_kernel: bool = False, cu_seqlens: Optional[Tensor] = None):
    """Chunked gated delta rule with per-channel decay.

    ``q, k, g [B, T, H, Dk]``, ``v [B, T, H, Dv]``, ``beta [B, T, H]``; returns
    ``(o [B, T, H, Dv], final_state [B, H, Dk, Dv] or None)``.  ``scale`` defaults
    to ``Dk ** -0.5``.  ``cu_seqlens`` (variable-length packing) is not supported.
    """
    if cu_seqlens is not None:
        raise NotImplementedError("chunk_kda: cu_seqlens (variable-length batches) is not supported")
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
        raise NotImplementedError("fused_recurrent_kda: cu_seqlens (variable-length batches) is not supported")
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
