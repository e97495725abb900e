"""fp32 restatement of the Kimi Delta Attention layer around the delta-rule core.

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

The reference's layer (models/daisy/attention_kimi.py:64-183) takes three pieces from the absent
third-party package flash-linear-attention (no version pinned, requirements.txt:20-21):
``ShortConvolution`` (attention_kimi.py:90-92, called at :155-158), ``rms_norm_gated``
(:41-62, called at :135-137) and ``chunk_kda`` (:133-134).  Their arithmetic is restated here from
the call sites and from the package's published behaviour:

* ``short_conv``: depthwise causal convolution over time (``kernel_size`` taps per channel, the
  weight of a grouped ``Conv1d``), optional bias, SiLU; the carried window ``[B, C, K]`` holds the
  last K inputs, zeros before the sequence starts; with ``cu_seqlens`` every packed sequence is
  convolved by itself.
* ``gated_rms_norm``: ``x * rsqrt(mean(x^2) + eps) * weight * sigmoid(gate)``, the
  ``FusedRMSNormGated(activation="sigmoid", eps=1e-5)`` that the reference's
  ``CompilableFusedRMSNormGated`` says it replaces (attention_kimi.py:41-42,103-104).

Pinned by ``tests/test_oracle_pins.py`` against library routines (``F.conv1d`` on an explicitly
padded sequence + ``F.silu``; ``F.rms_norm`` with a weight times ``torch.sigmoid``), brute-force
loops over taps on tiny inputs, and the invariant "two calls with the carried window == one call".
PARITY UNPINNED against flash-linear-attention itself: the layout of the carried window, the
placement of roundings in bf16 and -- for the gated norm -- whether ``rms_norm_gated`` called with
four positional arguments (attention_kimi.py:56) already applies a gate of its own before the
reference multiplies by ``sigmoid(gate)`` (:58-62) cannot be read from the reference tree.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .kda import kda_gate, kda_recurrent


def _conv_one(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], window: Optional[torch.Tensor],
              output_final_state: bool, activation: Optional[str]) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """One sequence ``x [T, C]`` (fp32), ``weight [C, K]``, ``window [C, K]`` or None."""
    T, C = x.shape
    K = weight.shape[1]
    before = window if window is not None else x.new_zeros(C, K)
    ext = torch.cat([before.transpose(0, 1), x], dim=0)              # [K + T, C]; ext[K + t] = x[t]
    y = x.new_zeros(T, C) if bias is None else bias[None, :].expand(T, C).clone()
    for j in range(K):                                               # tap j multiplies the input K-1-j steps back
        y = y + weight[None, :, j] * ext[1 + j: 1 + j + T]                # ext[1 + j + t] is the input at t - (K-1) + j
    if activation == "silu":
        y = y * torch.sigmoid(y)
    new_window = ext[-K:].transpose(0, 1).contiguous() if output_final_state else None
    return y, new_window


def short_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               cache: Optional[torch.Tensor] = None, output_final_state: bool = False,
               cu_seqlens: Optional[torch.Tensor] = None, activation: Optional[str] = "silu"):
    """``ShortConvolution.forward`` as called at models/daisy/attention_kimi.py:155-158.

    ``x [B, T, C]``; ``weight [C, 1, K]`` or ``[C, K]``; ``cache [B, C, K]`` (``[N, C, K]`` with
    ``cu_seqlens [N + 1]``, which needs ``B == 1``).  fp32 arithmetic; returns
    ``(y [B, T, C] fp32, new cache fp32 or None)``.
    """
    xf = x.float()
    w = weight.float().reshape(weight.shape[0], -1)
    b = None if bias is None else bias.float()
    B, T, C = xf.shape
    if cu_seqlens is None:
        spans = [(i, 0, T) for i in range(B)]
    else:
        assert B == 1
        cu = [int(v) for v in cu_seqlens.tolist()]
        spans = [(0, cu[i], cu[i + 1]) for i in range(len(cu) - 1)]
    y = torch.zeros_like(xf)
    windows = []
    for n, (row, s, e) in enumerate(spans):
        win = None if cache is None else cache[n].float()
        y_n, w_n = _conv_one(xf[row, s:e], w, b, win, output_final_state, activation)
        y[row, s:e] = y_n
        windows.append(w_n)
    return y, (torch.stack(windows, 0) if output_final_state else None)


def gated_rms_norm(x: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """``o_norm(o, gate)`` of the layer (models/daisy/attention_kimi.py:41-62,135-137) in fp64 -> fp32."""
    xd, gd, wd = x.double(), gate.double(), weight.double()
    y = xd / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + eps) * wd / (1.0 + torch.exp(-gd))
    return y.float()


def kimi_layer_forward(x: torch.Tensor, p: dict, num_heads: int, head_dim: int, conv_size: int = 4,
                       ve: Optional[torch.Tensor] = None, g_ve: Optional[float] = None,
                       cu_seqlens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``KimiLinearSelfAttention._forward_core`` without a cache (models/daisy/attention_kimi.py:141-185).

    ``p`` maps the reference's parameter names (``q_proj.weight``, ``q_conv1d.weight``, ``f_proj.0.weight``,
    ``f_proj.1.weight``, ``b_proj.weight``, ``A_log``, ``dt_bias``, ``g_proj.0.weight``, ``g_proj.1.weight``,
    ``g_proj.1.bias``, ``o_norm.weight``, ``o_proj.weight`` ...) to tensors.  The projections run in the
    parameters' dtype, as in the reference (bf16 there); everything between them in fp32.  Value heads may
    be wider than key heads (``head_v_dim = head_dim * expand_v``, attention_kimi.py:80): their width is read
    off the value projection.
    """
    lin = torch.nn.functional.linear
    B, T, _ = x.shape
    H, D = num_heads, head_dim
    Dv = p["v_proj.weight"].shape[0] // H
    x = x.to(p["q_proj.weight"].dtype)
    q, _ = short_conv(lin(x, p["q_proj.weight"]), p["q_conv1d.weight"], cu_seqlens=cu_seqlens)
    k, _ = short_conv(lin(x, p["k_proj.weight"]), p["k_conv1d.weight"], cu_seqlens=cu_seqlens)
    v, _ = short_conv(lin(x, p["v_proj.weight"]), p["v_conv1d.weight"], cu_seqlens=cu_seqlens)
    q, k, v = q.view(B, T, H, D), k.view(B, T, H, D), v.view(B, T, H, Dv)
    if g_ve is not None:
        gx = torch.sigmoid(torch.as_tensor(g_ve, dtype=torch.float32))
        v = gx * v + (1.0 - gx) * ve.float().view_as(v)
    g = kda_gate(lin(lin(x, p["f_proj.0.weight"]), p["f_proj.1.weight"]).float(), p["A_log"], D, p["dt_bias"])
    beta = torch.sigmoid(lin(x, p["b_proj.weight"])).float()
    if cu_seqlens is None:
        o, _ = kda_recurrent(q, k, v, g, beta, use_qk_l2norm=True)
    else:
        cu = [int(c) for c in cu_seqlens.tolist()]
        o = torch.zeros(B, T, H, Dv)
        for s, e in zip(cu[:-1], cu[1:]):
            if e > s:
                o[:, s:e], _ = kda_recurrent(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e], use_qk_l2norm=True)
    gate = lin(lin(x, p["g_proj.0.weight"]), p["g_proj.1.weight"], p["g_proj.1.bias"]).view(B, T, H, Dv)
    o = gated_rms_norm(o, gate, p["o_norm.weight"])
    return lin(o.reshape(B, T, H * Dv).to(p["o_proj.weight"].dtype), p["o_proj.weight"])
