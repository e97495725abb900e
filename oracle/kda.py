"""Naive fp32 Kimi Delta Attention recurrence and its gate.

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

The chunked kernel the reference calls (``fla.ops.kda.chunk_kda`` at
models/daisy/attention_kimi.py:133-134) lives in an absent third-party package
(flash-linear-attention, no version pinned in requirements.txt:20-21); its
published algorithm is the gated delta rule with a per-channel decay:

    S <- diag(exp(g_t)) S
    S <- S + beta_t k_t (v_t - S^T k_t)^T
    o_t = scale * S^T q_t

with ``S`` of shape ``[Dk, Dv]`` per (batch, head), q and k L2-normalised over
Dk when ``use_qk_l2norm_in_kernel=True``.  PARITY UNPINNED for three
conventions the reference tree does not show: default ``scale`` (Dk**-0.5
here), the L2-norm epsilon (``x / sqrt(sum(x^2) + 1e-6)`` here) and internal
rounding points.  All three are explicit arguments.
"""
from __future__ import annotations

from typing import Optional

import torch


def l2norm(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).sum(dim=-1, keepdim=True) + eps)


def kda_gate(g: torch.Tensor, A_log: torch.Tensor, head_k_dim: int,
             g_bias: Optional[torch.Tensor] = None, beta: float = 1.0, threshold: float = 20.0) -> torch.Tensor:
    """``-exp(A_log[h]) * softplus(g + bias)`` in fp32, cast back to ``g.dtype``.

    models/daisy/fla_custom_ops.py:71-103.  ``g`` is ``[..., H*Dk]``; the result is
    ``[..., H, Dk]``.  ``A_log`` has H elements; ``g_bias`` may be ``[H*Dk]``,
    ``[H, Dk]``, ``[1, 1, H, Dk]`` or ``[H]`` (fla_custom_ops.py:54-66).
    softplus is linear above ``threshold`` (``beta * x > threshold``).
    """
    H = g.shape[-1] // head_k_dim
    x = g.float().reshape(*g.shape[:-1], H, head_k_dim)
    if g_bias is not None:
        b = g_bias.float()
        b = b.reshape(H, 1).expand(H, head_k_dim) if b.numel() == H else b.reshape(H, head_k_dim)
        x = x + b
    bx = x * beta
    sp = torch.where(bx > threshold, x, torch.log1p(torch.exp(torch.minimum(bx, torch.tensor(threshold)))) / beta)
    a = -torch.exp(A_log.float().reshape(H, 1))
    return (a * sp).to(g.dtype)


def kda_recurrent(q, k, v, g, beta, scale: Optional[float] = None,
                  initial_state: Optional[torch.Tensor] = None, use_qk_l2norm: bool = True,
                  l2_eps: float = 1e-6, dtype=torch.float32):
    """Token-by-token recurrence; q, k, g ``[B, T, H, Dk]``, v ``[B, T, H, Dv]``,
    beta ``[B, T, H]``; returns ``o [B, T, H, Dv]`` and the final state
    ``[B, H, Dk, Dv]`` (both in ``dtype``, fp32 by default, fp64 for pinning), on the inputs' device
    (the same library calls either way; full-size checks run the loop on the GPU's fp32 units).
    """
    B, T, H, Dk = q.shape
    Dv = v.shape[-1]
    if scale is None:
        scale = Dk ** -0.5
    qf, kf = q.to(dtype), k.to(dtype)
    if use_qk_l2norm:
        qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + l2_eps)
        kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + l2_eps)
    vf, gf, bf = v.to(dtype), g.to(dtype), beta.to(dtype)
    S = torch.zeros(B, H, Dk, Dv, dtype=dtype, device=q.device) if initial_state is None else initial_state.to(dtype).clone()
    o = torch.empty(B, T, H, Dv, dtype=dtype, device=q.device)
    for t in range(T):
        S = S * torch.exp(gf[:, t])[..., None]                      # decay rows of S
        pred = torch.einsum("bhkv,bhk->bhv", S, kf[:, t])            # S^T k_t
        delta = (vf[:, t] - pred) * bf[:, t][..., None]              # beta_t (v_t - S^T k_t)
        S = S + torch.einsum("bhk,bhv->bhkv", kf[:, t], delta)
        o[:, t] = scale * torch.einsum("bhkv,bhk->bhv", S, qf[:, t])
    return o, S
