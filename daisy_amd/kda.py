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


def _bf16(t: Tensor) -> Tensor:
    return t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)


def _cu(cu_seqlens: Optional[Tensor], like: Tensor) -> Optional[Tensor]:
    """The packed-sequence bounds as the kernels read them: int32, contiguous, on the tensors' GPU.
    A device tensor is passed through without a synchronisation; the host never looks at the values."""
    if cu_seqlens is None:
        return None
    return cu_seqlens.to(device=like.device, dtype=torch.int32).contiguous()


def chunk_kda(q: Tensor, k: Tensor, v: Tensor, g: Tensor, beta: Tensor, scale: Optional[float] = None,
              initial_state: Optional[Tensor] = None, output_final_state: bool = False,
              use_qk_l2norm_in_kernel: bool = False, cu_seqlens: Optional[Tensor] = None):
    """Chunked gated delta rule with per-channel decay.

    ``q, k, g [B, T, H, Dk]``, ``v [B, T, H, Dv]``, ``beta [B, T, H]``; returns
    ``(o [B, T, H, Dv], final_state [B, H, Dk, Dv] or None)``.  ``scale`` defaults
    to ``Dk ** -0.5``.  With ``cu_seqlens [N + 1]`` the batch is 1 and holds N sequences packed
    along T, each with its own state (``initial_state`` / ``final_state [N, H, Dk, Dv]``); the
    bounds are handed to the kernels as they are (one call, as at
    models/daisy/attention_kimi.py:133-134), sequence boundaries are resolved on the device.
    """
    o, final = ops.kda_chunk_fwd(_bf16(q), _bf16(k), _bf16(v), g, beta, scale=scale, initial_state=initial_state,
                                 output_final_state=output_final_state,
                                 use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, cu_seqlens=_cu(cu_seqlens, q))
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
    o, final = ops.kda_recurrent_fwd(_bf16(q), _bf16(k), _bf16(v), g, beta, scale=scale, initial_state=initial_state,
                                     output_final_state=output_final_state or inplace_state,
                                     use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, inplace_state=inplace_state,
                                     cu_seqlens=_cu(cu_seqlens, q))
    return o.to(v.dtype), (final if (output_final_state or inplace_state) else None)


def fused_kda_gate(g: Tensor, A_log: Tensor, head_k_dim: int, g_bias: Optional[Tensor] = None,
                   b: Optional[Tensor] = None, beta: float = 1.0, threshold: float = 20.0):
    """``-exp(A_log) * softplus(g + bias)`` reshaped to ``[..., H, Dk]``; with ``b`` also ``sigmoid(b)``."""
    y = ops.kda_gate_fwd(g, A_log, head_k_dim, g_bias, beta, threshold)
    return y if b is None else (y, torch.sigmoid(b.to(dtype=g.dtype)))
