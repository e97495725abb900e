"""Kimi Delta Attention layer with the reference's module layout (models/daisy/attention_kimi.py:64-200).

Same parameters and names as the reference's ``KimiLinearSelfAttention`` (``q_proj``, ``k_proj``,
``v_proj``, ``q_conv1d.weight`` ..., ``f_proj``, ``b_proj``, ``A_log``, ``dt_bias``, ``g_proj``,
``o_norm.weight``, ``o_proj``), the interface of ``AttentionProtocol``
(models/daisy/attention_protocol.py:4-42) -- the reference's own ``forward`` / ``prefill`` /
``step`` pass five arguments to a four-argument ``_forward_core`` and use an undefined
``sa_lambdas``, so they cannot run as written -- and the arithmetic of ``_forward_core``:

    q, k, v = silu(causal_conv4(proj(x)))          short depthwise convolutions, state kept for decode
    g       = -exp(A_log) * softplus(f_proj(x) + dt_bias)       (``fused_kda_gate``)
    beta    = sigmoid(b_proj(x)) in fp32
    o, S    = chunk_kda(q, k, v, g, beta, S0, use_qk_l2norm_in_kernel=True)
    y       = o_proj(rms_norm(o) * o_norm.weight * sigmoid(g_proj(x)))

The delta-rule core runs on the HIP kernels (``chunk_kda`` for sequences, ``fused_recurrent_kda``
with the state updated in place for single-token steps), and so do the four-tap convolutions
with their SiLU and the gated norm (one streaming kernel each, ``daisy_short_conv_fwd`` and
``daisy_gated_rmsnorm_fwd``; like every op of this package they run on the GPU only and raise
for CPU tensors); the projections are library GEMMs.  Three pieces of the reference come from the absent
``flash-linear-attention`` package and are restated from their documented behaviour, not pinned
against it: ``ShortConvolution`` (depthwise causal conv + SiLU with a ``[B, C, K]`` state) and
the gated RMS norm (``FusedRMSNormGated(activation="sigmoid", eps=1e-5)``, the module the
reference's ``CompilableFusedRMSNormGated`` stands in for), and ``chunk_kda``'s conventions.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import ops
from . import attention as _attention
from .attention import step_linear
from .kda import chunk_kda, fused_kda_gate, fused_recurrent_kda


class ShortConvolution(nn.Module):
    """Depthwise causal 1-D convolution + SiLU over ``[B, T, C]`` with a carried window.

    ``weight [C, 1, K]`` like a grouped ``nn.Conv1d``.  ``cache [B, C, K]`` holds the last K
    inputs (zeros before the sequence starts); the returned cache continues the sequence.
    """

    def __init__(self, hidden_size: int, kernel_size: int, activation: str = "silu", bias: bool = False,
                 dtype=torch.bfloat16):
        super().__init__()
        assert activation == "silu"
        self.hidden_size, self.kernel_size = hidden_size, kernel_size
        w = torch.empty(hidden_size, 1, kernel_size, dtype=dtype)
        nn.init.kaiming_uniform_(w, a=5 ** 0.5)
        self.weight = nn.Parameter(w)
        self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=dtype)) if bias else None

    def forward(self, x: Tensor, cache: Optional[Tensor] = None, output_final_state: bool = False,
                cu_seqlens: Optional[Tensor] = None, inplace_cache: bool = False) -> Tuple[Tensor, Optional[Tensor]]:
        """One streaming kernel (``ops.short_conv``); tensors must be bf16 on the GPU, like every op of
        this package.  ``cu_seqlens``: sequences packed along T of a batch of one -- the window does not
        reach across a boundary and the caches are ``[N, C, K]``; the bounds stay on the device.
        ``inplace_cache`` (a few steps at a time): the window is updated inside ``cache`` and that
        tensor is returned, so that its address stays the same from step to step."""
        if cu_seqlens is not None:
            cu_seqlens = cu_seqlens.to(device=x.device, dtype=torch.int32).contiguous()
        return ops.short_conv(x, self.weight, self.bias, cache, output_final_state, "silu",
                              inplace_cache=inplace_cache, cu_seqlens=cu_seqlens)


class GatedRMSNorm(nn.Module):
    """``rms_norm(x, eps) * weight * sigmoid(gate)`` over the last dim (fp32 statistics)."""

    def __init__(self, hidden_size: int, eps: float = 1e-5, dtype=torch.bfloat16):
        super().__init__()
        self.hidden_size, self.eps = hidden_size, eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype))

    def forward(self, x: Tensor, gate: Tensor) -> Tensor:
        return ops.gated_rmsnorm(x, gate, self.weight, self.eps)


def _project(lin: nn.Linear, x: Tensor) -> Tensor:
    """``lin(x)``; a bias-free projection of a decode step's few rows reads its weights through the few-rows kernel."""
    if lin.bias is None:
        return step_linear(x, lin.weight)
    return lin(x)


class KimiLinearSelfAttention(nn.Module):
    """Linear-attention layer on the KDA kernels; see the module docstring.

    ``ve`` is accepted for interface compatibility; it is mixed into v as in ``CausalSelfAttention``
    (``sigmoid(g_ve) * v + (1 - sigmoid(g_ve)) * ve``) when ``receives_ve`` is set and ignored
    otherwise (the reference leaves this as a TODO).  A two-dimensional ``attn_mask [B, S]`` is a
    padding mask as in the reference (models/daisy/attention_kimi.py:150-154, 1 = token,
    0 = padding): the tokens are packed into one row, every sequence runs by itself
    (``cu_seqlens``), and the padded positions of the result are zero.  Any other ``attn_mask``
    (window descriptors, dense attention masks) is ignored: the recurrence is causal by
    construction and a window does not apply.  ``block_mask`` must be None as in the reference.
    """

    def __init__(self, dim: int, num_heads: int, max_seq_len: int, head_dim: int, expand_v: float = 1.0,
                 mode: str = "chunk", use_short_conv: bool = True, allow_neg_eigval: bool = False, conv_size: int = 4,
                 conv_bias: bool = False, layer_idx: int = 0, receives_ve: bool = False):
        assert not allow_neg_eigval, "allow_neg_eigval is not supported"
        assert mode == "chunk", "mode must be 'chunk' (single-token steps use the recurrent kernel by themselves)"
        super().__init__()
        self.hidden_size, self.num_heads, self.head_dim = dim, num_heads, head_dim
        self.head_k_dim, self.head_v_dim = head_dim, int(head_dim * expand_v)
        # What the kernels under this layer serve, checked here rather than at the first call: key heads of up to
        # 128 channels (a multiple of 8), value heads of 32, 64, 128 or 256 columns (the delta-rule kernels take any
        # multiple of 8; the gated norm takes these four), convolutions of 2 to 4 taps, bf16 parameters (this
        # constructor makes them so).
        if not (8 <= self.head_k_dim <= 128 and self.head_k_dim % 8 == 0):
            raise ValueError(f"KimiLinearSelfAttention: head_dim {head_dim} not supported by the KDA kernels (a multiple of 8 up to 128)")
        if self.head_v_dim not in (32, 64, 128, 256):
            raise ValueError(f"KimiLinearSelfAttention: head_dim * expand_v = {self.head_v_dim} not supported (32, 64, 128 or 256)")
        if use_short_conv and not 2 <= conv_size <= 4:
            raise ValueError(f"KimiLinearSelfAttention: conv_size {conv_size} not supported by the convolution kernel (2 to 4)")
        self.key_dim, self.value_dim = num_heads * self.head_k_dim, num_heads * self.head_v_dim
        self.use_short_conv, self.conv_size, self.layer_idx = use_short_conv, conv_size, layer_idx
        bf = torch.bfloat16
        self.q_proj = nn.Linear(dim, self.key_dim, bias=False, dtype=bf)
        self.k_proj = nn.Linear(dim, self.key_dim, bias=False, dtype=bf)
        self.v_proj = nn.Linear(dim, self.value_dim, bias=False, dtype=bf)
        if use_short_conv:
            self.q_conv1d = ShortConvolution(self.key_dim, conv_size, bias=conv_bias, dtype=bf)
            self.k_conv1d = ShortConvolution(self.key_dim, conv_size, bias=conv_bias, dtype=bf)
            self.v_conv1d = ShortConvolution(self.value_dim, conv_size, bias=conv_bias, dtype=bf)
        self.f_proj = nn.Sequential(nn.Linear(dim, self.head_v_dim, bias=False, dtype=bf),
                                    nn.Linear(self.head_v_dim, self.key_dim, bias=False, dtype=bf))
        self.b_proj = nn.Linear(dim, num_heads, bias=False, dtype=bf)
        self.A_log = nn.Parameter(torch.log(torch.empty(num_heads, dtype=torch.float32).uniform_(1, 16)).view(1, 1, -1, 1))
        self.A_log._no_weight_decay = True
        self.dt_bias = nn.Parameter(torch.zeros(self.key_dim, dtype=torch.float32))
        self.dt_bias._no_weight_decay = True
        self.g_proj = nn.Sequential(nn.Linear(dim, self.head_v_dim, bias=False, dtype=bf),
                                    nn.Linear(self.head_v_dim, self.value_dim, bias=True, dtype=bf))
        self.o_norm = GatedRMSNorm(self.head_v_dim, eps=1e-5, dtype=bf)
        self.o_proj = nn.Linear(self.value_dim, dim, bias=False, dtype=bf)
        self.receives_ve = receives_ve
        self.g_ve = nn.Parameter(torch.tensor(0.0)) if receives_ve else None
        self._recurrent_state: Optional[Tensor] = None
        self._conv_state = None
        self._seen = 0
        # Buffers that held the states before a reset_history, by batch size: the next prompt's states
        # of that batch size are stored into them, so that the addresses a recorded decode step reads
        # and writes stay the same for the life of the module, also when calls of different batch
        # sizes alternate (a recorded step checks the addresses before every replay all the same).
        self._state_homes: dict = {}
        # The six projections that read the layer's input, stacked into one matrix for decode steps (see
        # _input_projections); rebuilt when one of the weights moves or changes.
        self._stacked_w: Optional[Tensor] = None
        self._stacked_key = None

    def replay_guard(self) -> tuple:
        """What a recorded decode step of this layer depends on besides the tensors it updates in place: the stacked
        copy of the input projections is a snapshot, so a recording is good for as long as the six weights keep their
        addresses and versions (``core.GraphedStep`` compares this before every replay and records again otherwise)."""
        lins = (self.q_proj, self.k_proj, self.v_proj, self.f_proj[0], self.g_proj[0], self.b_proj)
        return tuple((l.weight.data_ptr(), l.weight._version) for l in lins)

    def _input_projections(self, x: Tensor):
        """``q_proj(x), k_proj(x), v_proj(x), f_proj[0](x), g_proj[0](x), b_proj(x)``.  For the few rows of a decode
        step (no autograd, bf16 on the GPU) the six weight matrices are kept stacked and read by ONE launch of the
        few-rows kernel instead of six; its rows are computed one by one, so every output equals the separate call's
        bit for bit.  The stack (as large as the six weights) is made outside stream capture and follows the
        parameters' addresses and versions."""
        lins = (self.q_proj, self.k_proj, self.v_proj, self.f_proj[0], self.g_proj[0], self.b_proj)
        rows = x.numel() // x.shape[-1]
        fused = (rows <= _attention.STEP_ROWS_KERNEL_MAX and x.is_cuda and x.dtype == torch.bfloat16
                 and not (torch.is_grad_enabled() and (x.requires_grad or any(l.weight.requires_grad for l in lins)))
                 and all(l.bias is None and l.weight.dtype == torch.bfloat16 for l in lins))
        if fused:
            key = self.replay_guard()
            if key != self._stacked_key:
                if torch.cuda.is_current_stream_capturing():
                    fused = False          # not the moment to build it: the separate launches are recorded
                else:
                    with torch.no_grad():
                        w = torch.cat([l.weight for l in lins], 0)
                        if w.shape[0] % 8:  # whole 16-byte pieces per output row of a batch
                            w = torch.cat([w, w.new_zeros(8 - w.shape[0] % 8, w.shape[1])], 0)
                    self._stacked_w, self._stacked_key = w.contiguous(), key
        if fused and ops.linear_rows_ok(x, self._stacked_w):
            sizes = [l.weight.shape[0] for l in lins]
            y = ops.linear_rows(x, self._stacked_w)
            return y[..., :sum(sizes)].split(sizes, dim=-1)
        return tuple(_project(l, x) for l in lins)

    def _apply(self, fn, recurse=True):
        # The decay parameters stay fp32 under module-wide casts, as the reference creates them.
        super()._apply(fn, recurse)
        for name in ("A_log", "dt_bias"):
            prm = getattr(self, name)
            if prm.dtype != torch.float32:
                prm.data = prm.data.float()
        return self

    # step() keeps its own recurrent and convolution states; the k_ctx / v_ctx arguments are not read.
    uses_kv_context = False

    def reset_history(self):
        if self._recurrent_state is not None:
            self._state_homes[self._recurrent_state.shape[0]] = \
                (self._recurrent_state,) + tuple(self._conv_state or (None, None, None))
        self._recurrent_state = None
        self._conv_state = None
        self._seen = 0

    def state_tensors(self):
        """The tensors a decode step updates in place (recurrent state, convolution windows)."""
        held = (self._recurrent_state,) + tuple(self._conv_state or ())
        return [t for t in held if t is not None]

    @staticmethod
    def _store(home: Optional[Tensor], fresh: Optional[Tensor]) -> Optional[Tensor]:
        """``fresh`` itself, or ``home`` holding its values when that buffer fits."""
        if fresh is None or home is None or home is fresh:
            return fresh
        if home.shape == fresh.shape and home.dtype == fresh.dtype and home.device == fresh.device:
            home.copy_(fresh)
            return home
        return fresh

    def _core(self, x: Tensor, ve: Optional[Tensor], use_cache: bool, attn_mask=None) -> Tensor:
        B0, S0, _ = x.shape
        H, Dk, Dv = self.num_heads, self.head_k_dim, self.head_v_dim
        x = x.to(self.q_proj.weight.dtype)
        indices = cu_seqlens = None
        if isinstance(attn_mask, Tensor) and attn_mask.ndim == 2:
            # get_unpad_data of the reference's dependency, restated: positions of the tokens in the
            # flattened batch and the running sequence lengths.
            keep = attn_mask[:, -S0:].to(torch.bool)
            indices = torch.nonzero(keep.flatten(), as_tuple=False).flatten()
            cu_seqlens = F.pad(torch.cumsum(keep.sum(-1), 0), (1, 0)).to(torch.int32)
            x = x.flatten(0, 1)[indices].unsqueeze(0)
            if ve is not None:
                ve = ve.reshape(B0 * S0, -1)[indices].unsqueeze(0)
        B, T, _ = x.shape
        state = self._recurrent_state if use_cache else None
        convs = self._conv_state if (use_cache and self._conv_state is not None) else (None, None, None)
        q_lin, k_lin, v_lin, f_low, g_low, b_lin = self._input_projections(x)
        if self.use_short_conv:
            # a decode step shifts its windows in place (same tensors, same addresses, every step)
            shift = (use_cache and T == 1 and cu_seqlens is None
                     and all(c is not None and c.dtype == torch.bfloat16 and c.is_contiguous() for c in convs))
            q, cq = self.q_conv1d(q_lin, convs[0], use_cache, cu_seqlens, shift)
            k, ck = self.k_conv1d(k_lin, convs[1], use_cache, cu_seqlens, shift)
            v, cv = self.v_conv1d(v_lin, convs[2], use_cache, cu_seqlens, shift)
        else:
            q, k, v = F.silu(q_lin), F.silu(k_lin), F.silu(v_lin)
            cq = ck = cv = None
        q, k, v = q.view(B, T, H, Dk), k.view(B, T, H, Dk), v.view(B, T, H, Dv)
        if self.receives_ve:
            torch._assert(ve is not None, "ve must be provided when receives_ve=True")
            g_x = torch.sigmoid(self.g_ve).to(v.dtype)
            v = g_x * v + (1.0 - g_x) * ve.view_as(v).to(v.dtype)
        g = fused_kda_gate(_project(self.f_proj[1], f_low), self.A_log, Dk, self.dt_bias)
        beta = torch.sigmoid(b_lin).to(torch.float32)
        if use_cache and T == 1 and state is not None and cu_seqlens is None:
            o, state = fused_recurrent_kda(q, k, v, g, beta, initial_state=state, use_qk_l2norm_in_kernel=True,
                                           inplace_state=True)
        else:
            o, state = chunk_kda(q, k, v, g, beta, initial_state=state, output_final_state=use_cache,
                                 use_qk_l2norm_in_kernel=True, cu_seqlens=cu_seqlens)
        if use_cache:
            homes = self._state_homes.get(state.shape[0], (None, None, None, None))
            self._recurrent_state = self._store(homes[0], state)
            self._conv_state = tuple(self._store(h, c) for h, c in zip(homes[1:], (cq, ck, cv)))
            self._state_homes[state.shape[0]] = (self._recurrent_state,) + self._conv_state
            self._seen += T
        # (contiguous rows: the library adds the bias inside the product then, as it does for the reference's tensors)
        gate = self.g_proj[1](g_low.contiguous()).view(B, T, H, Dv)
        o = self.o_norm(o.to(gate.dtype), gate)
        y = _project(self.o_proj, o.reshape(B, T, H * Dv))
        if indices is not None:   # back to the padded layout, zeros where the mask was 0
            padded = y.new_zeros(B0 * S0, y.size(-1))
            padded[indices] = y[0]
            y = padded.view(B0, S0, -1)
        return y

    def forward(self, x: Tensor, ve: Optional[Tensor], attn_mask=None, block_mask=None) -> Tensor:
        assert block_mask is None, "block_mask not supported for KimiLinearSelfAttention"
        return self._core(x, ve, use_cache=False, attn_mask=attn_mask)

    def prefill(self, x: Tensor, ve: Optional[Tensor], attn_mask=None, debug: bool = False):
        """Runs the prompt and keeps the recurrent and convolution states; there is no K/V to cache."""
        return self._core(x, ve, use_cache=True, attn_mask=attn_mask), None, None

    def step(self, x: Tensor, k_ctx, v_ctx, pos: int, ve: Optional[Tensor], window: Optional[int]):
        torch._assert(x.size(1) == 1, "step() requires single position only")
        return self._core(x, ve, use_cache=True), None, None
