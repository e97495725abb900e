"""Prefill / step glue over a Daisy model (models/daisy/daisy_core.py:294-370), cache-aware.

The reference's ``DaisyCore.prefill`` builds a dense ``[1, 1, T, T]`` mask, stacks every layer's
keys and values into ``kv [2, L, B, H, T, D]`` and hands that to ``KVCache.bulk_write_packed``;
``DaisyCore.step`` takes one token of one sequence.  The two functions here walk the same
model attributes (``embed``, ``blocks``, ``skip_map``, ``skip_weights``, ``ve_module_map`` /
``compute_value_embeddings``, ``lm_head_w``, ``window_size``, ``attn_window_size``,
``eos_token_id``) with the same arithmetic, but

* pass the window / document mask as a descriptor (no T x T tensor, no T <= 46340 cap),
* write each layer's keys and values straight into the ring cache as the layer finishes
  (nothing of size ``L * T`` is ever stacked; a prompt shorter than the ring is written into its
  slots by the pre-attention kernel itself, with no copy at all), and
* accept a batch of sequences (the cache has a batch dimension; the reference pins B = 1).

They work on the reference's ``DaisyCore`` once its blocks hold this package's
``CausalSelfAttention``, and on any module with the same attributes.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import dataclasses

import torch
import torch.nn.functional as F
from torch import Tensor

from .attention import CausalSelfAttention, WindowMask, step_linear, build_window_mask
from .functional import norm
from .kv_cache import KVCache


def _value_embeddings(model, ids: Tensor) -> Dict[int, Tensor]:
    if hasattr(model, "compute_value_embeddings"):
        return model.compute_value_embeddings(ids)
    return {i: m(ids) for i, m in getattr(model, "ve_module_map", {}).items()}


def _mask_for(model, input_seq: Tensor) -> WindowMask:
    window = getattr(model, "window_size", None)
    if input_seq.size(0) == 1:
        return build_window_mask(input_seq, window, model.eos_token_id)
    # One descriptor serves the whole batch, so document boundaries (which differ per row)
    # cannot be expressed: a batch must not contain the end-of-sequence token.
    torch._assert(bool((input_seq != model.eos_token_id).all()),
                  "batched prefill needs prompts without the end-of-sequence token")
    return WindowMask(window, None)


@torch.no_grad()
def prefill(model, input_seq: Tensor, cache: Optional[KVCache] = None, debug: bool = False
            ) -> Tuple[Tensor, Optional[Tensor]]:
    """``DaisyCore.prefill`` (daisy_core.py:325-370) for ``input_seq [B, T]``.

    With ``cache`` the keys/values of every layer go straight into it (``cache.t`` becomes T) and
    ``(logits [B, V], None)`` is returned; without, ``(logits, kv [2, L, B, H, T, D])`` as the
    reference does.
    """
    assert input_seq.ndim == 2
    B, T = input_seq.shape
    L = len(model.blocks)
    x = x0 = norm(model.embed(input_seq))
    skip_map, skip_weights = model.skip_map, model.skip_weights
    ve_map = _value_embeddings(model, input_seq)
    attn_mask = _mask_for(model, input_seq)
    k_list: List[Optional[Tensor]] = []
    v_list: List[Optional[Tensor]] = []
    skip_connections = []
    for i in range(L):
        if i in skip_map:
            gate = torch.sigmoid(skip_weights[skip_map[i]])
            x = x * gate + (1 - gate) * skip_connections[skip_map[i]]
        # A prompt that fits the ring without wrapping (T <= W - 1: position p goes to slot p) is
        # written there by the pre-attention kernel itself; the attention kernel then reads its keys
        # and values from the ring and nothing is copied afterwards.
        attn = getattr(model.blocks[i], "attn", None)
        direct = (cache is not None and cache.dtype == torch.bfloat16 and T <= cache.W - 1
                  and isinstance(attn, CausalSelfAttention) and attn._fused_prep_ok())
        layer_mask = attn_mask
        if direct:
            # the destination rides on the mask descriptor, which a block hands to its attention untouched
            layer_mask = dataclasses.replace(attn_mask, kv_out=(cache.k[i][:, :, :T].transpose(1, 2),
                                                                cache.v[i][:, :, :T].transpose(1, 2)))
        x, k, v = model.blocks[i].prefill(x, ve_map.get(i), x0, attn_mask=layer_mask, debug=debug)
        skip_connections.append(x)
        if cache is not None:
            if k is not None and not direct:
                cache.bulk_write_layer(i, k, v, T)
        else:
            k_list.append(k)
            v_list.append(v)
    x = norm(x)
    logits = F.linear(x[:, -1].bfloat16(), model.lm_head_w.bfloat16()).float()
    if cache is not None:
        cache.t = T
        cache._staged = [False] * cache.L
        return logits, None
    H, D = model.attn_num_heads, model.attn_head_dim
    zeros = None
    K, V = [], []
    for k, v in zip(k_list, v_list):
        if k is None:
            if zeros is None:
                zeros = torch.zeros(B, H, T, D, device=x.device, dtype=x.dtype)
            k = v = zeros
        K.append(k)
        V.append(v)
    return logits, torch.stack([torch.stack(K, dim=0), torch.stack(V, dim=0)], dim=0)


@torch.no_grad()
def step(model, token_ids: Tensor, cache: KVCache) -> Tensor:
    """``DaisyCore.step`` (daisy_core.py:294-323) for one new token per sequence, ``token_ids [B]``
    (or a 0-dim tensor when B = 1), at position ``cache.t``.

    Each attention layer streams its ring in place and appends the new row itself (bf16 cache and
    this package's attention), or gets the chronological view and the row is written here.
    Advances the cache; returns ``logits [B, V]``.
    """
    logits = _walk_step(model, token_ids, cache, cache.t)
    cache.advance()
    return logits


def _walk_step(model, token_ids: Tensor, cache: KVCache, pos, status: Optional[Tensor] = None) -> Tensor:
    """The layer walk of ``step`` at position ``pos`` (a host int, or a one-element int32 device
    tensor when the walk is being recorded for replay); leaves ``cache.advance()`` to the caller.
    ``status``: the int32 word in which the attention kernels report a device position they cannot use."""
    token_ids = token_ids.reshape(-1, 1)
    B = token_ids.size(0)
    torch._assert(B == cache.B, "token batch does not match the cache")
    on_device = isinstance(pos, Tensor)
    L = len(model.blocks)
    x = x0 = norm(model.embed(token_ids))
    skip_map, skip_weights = model.skip_map, model.skip_weights
    ve_map = _value_embeddings(model, token_ids)
    window = getattr(model, "attn_window_size", cache.W)
    in_place = cache.dtype in (torch.bfloat16, torch.float16)
    skip_connections = []
    for i in range(L):
        if i in skip_map:
            gate = torch.sigmoid(skip_weights[skip_map[i]])
            x = x * gate + (1 - gate) * skip_connections[skip_map[i]]
        blk = model.blocks[i]
        if getattr(blk, "attn", None) is None or not getattr(blk.attn, "uses_kv_context", True):
            k_ctx = v_ctx = None        # no attention, or one that keeps its own state (KDA layers)
        elif in_place and getattr(blk.attn, "accepts_ring_context", False):
            k_ctx = v_ctx = cache.ring(i)
            k_ctx.status = status
        else:
            torch._assert(not on_device, "a recorded step needs attention layers that take the ring in place")
            k_ctx, v_ctx = cache.view(i)
        x, k_new, v_new = blk.step(x, ve_map.get(i), x0, k_ctx, v_ctx, pos, window)
        skip_connections.append(x)
        if k_new is not None and not cache._staged[i]:
            torch._assert(not on_device, "a recorded step needs attention layers that write the ring themselves")
            cache.write(i, k_new.to(cache.dtype), v_new.to(cache.dtype))
    x = norm(x)
    return step_linear(x.flatten(end_dim=1).bfloat16(), model.lm_head_w.bfloat16()).float()


class GraphedStep:
    """``step(model, tokens, cache)`` recorded once as a HIP graph and replayed for every later token.

    A decode step of a small model is a few hundred short kernels, and launching them one by one
    from Python costs more than running them.  Nothing in the recorded walk depends on the host's
    idea of the position: the token ids sit in a fixed input buffer, and the position sits in a
    device counter that the pre-attention and decode kernels read when they run and that the last
    node of the graph increments.

    Needs a bf16 or fp16 cache whose ring size equals the model's attention window and attention layers
    that take the ring in place with the fused pre-attention kernel (otherwise recording raises).
    The returned logits are a buffer that the next call overwrites.  Rotary tables are fixed when
    the step is recorded: positions up to their row count can be replayed.
    """

    def __init__(self, model, cache: KVCache):
        torch._assert(cache.dtype in (torch.bfloat16, torch.float16), "a recorded step needs a bf16 or fp16 cache")
        self.model, self.cache = model, cache
        dev = cache.k.device
        self.tokens = torch.zeros(cache.B, dtype=torch.long, device=dev)
        self.pos = torch.zeros(1, dtype=torch.int32, device=dev)
        self._pos_host: Optional[int] = None      # what self.pos holds, None = unknown
        self._graph: Optional[torch.cuda.CUDAGraph] = None
        self._logits: Optional[Tensor] = None
        self._recorded_addresses: Optional[tuple] = None
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)   # raised by the kernels, see check()
        tables = [blk.attn.rotary.cos.shape[0] for blk in model.blocks
                  if getattr(blk, "attn", None) is not None and hasattr(blk.attn, "rotary")]
        self.max_positions = min(tables) if tables else None

    def _stateful_tensors(self) -> List[Tensor]:
        """State that layers keep by themselves (the KDA layer's recurrent state and convolution windows)."""
        return [t for blk in self.model.blocks if hasattr(getattr(blk, "attn", None), "state_tensors")
                for t in blk.attn.state_tensors()]

    def _addresses(self) -> tuple:
        """Every address the recorded launches carry besides the parameters: the ring and the layers' own state; and
        what layers that read a snapshot of their parameters say the snapshot depends on (``replay_guard``)."""
        guards = tuple(blk.attn.replay_guard() for blk in self.model.blocks if hasattr(getattr(blk, "attn", None), "replay_guard"))
        return (self.cache.k.data_ptr(), self.cache.v.data_ptr()) + tuple(t.data_ptr() for t in self._stateful_tensors()) + guards

    def check(self) -> None:
        """Raises what the kernels of the replayed steps reported (a position past the rotary tables).
        Reads one word from the device, so it synchronises: call it after a run of steps, not per step."""
        from . import ops
        ops.raise_for_status(self.status)

    def _body(self) -> Tensor:
        logits = _walk_step(self.model, self.tokens, self.cache, self.pos, self.status)
        self.pos.add_(1)
        return logits

    @torch.no_grad()
    def _record(self):
        dev = self.cache.k.device
        # One eager pass on a side stream first (library handles, workspaces, the allocator's pools);
        # in the ring it writes the same row the first replay writes again.
        # Layers that keep their own state (KDA) would advance it twice: it is put back afterwards.
        stateful = self._stateful_tensors()
        saved = [t.clone() for t in stateful]
        before = self._addresses()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            self._body()
        torch.cuda.current_stream(dev).wait_stream(side)
        for t, old in zip(stateful, saved):
            t.copy_(old)
        self.pos.fill_(self.cache.t)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._logits = self._body()
        self.cache._staged = [False] * self.cache.L    # recording ran no kernel
        # The graph carries raw addresses.  A layer that made a new state tensor during the walk (no
        # prefill before the first step, a window that could not be shifted in place) would leave the
        # graph pointing at memory that belongs to the capture: refuse to replay such a recording.
        self._recorded_addresses = self._addresses()
        if self._recorded_addresses != before:
            self._graph = None
            raise RuntimeError("a recorded step needs layers that update their state in place: run a prefill first "
                               "(the KDA layer creates its state there) and keep the cache's tensors")

    @torch.no_grad()
    def __call__(self, token_ids: Tensor) -> Tensor:
        cache = self.cache
        if self.max_positions is not None:
            torch._assert(cache.t < self.max_positions, f"Rotary buffers too small {self.max_positions} < {cache.t + 1}")
        self.tokens.copy_(token_ids.reshape(-1))
        if self._pos_host != cache.t:
            self.pos.fill_(cache.t)
        if self._graph is not None and self._addresses() != self._recorded_addresses:
            # A prefill of another batch size, a new cache tensor, a reset that moved a layer's state: the
            # recording points at memory that may have been freed.  Record again at the current addresses.
            self._graph = None
        if self._graph is None:
            self._record()
        self._graph.replay()
        cache.advance()
        self._pos_host = cache.t
        return self._logits


@torch.no_grad()
def generate_greedy(model, prompt_ids: Tensor, max_new_tokens: int, window: Optional[int] = None,
                    cache: Optional[KVCache] = None, record_steps: bool = False) -> Tensor:
    """Greedy continuation of a batch of equally long prompts ``[B, T]`` -> ``[B, max_new_tokens]``.

    Rows that produce the end-of-sequence token keep emitting it.  The cache (bf16 ring of
    ``window`` slots, default the model's window) is created unless given.  ``record_steps``: the
    decode step is recorded once (``GraphedStep``) and replayed for every token.
    """
    assert prompt_ids.ndim == 2 and prompt_ids.size(1) > 0 and max_new_tokens > 0
    B = prompt_ids.size(0)
    dev = prompt_ids.device
    if cache is None:
        W = window if window is not None else model.attn_window_size
        cache = KVCache(L=len(model.blocks), B=B, H=model.attn_num_heads, W=W, D=model.attn_head_dim,
                        device=dev, dtype=torch.bfloat16)
    vocab = model.embed.num_embeddings
    logits, _ = prefill(model, prompt_ids, cache)
    one_step = GraphedStep(model, cache) if record_steps else (lambda tokens: step(model, tokens, cache))
    done = torch.zeros(B, dtype=torch.bool, device=dev)
    eos = torch.tensor(model.eos_token_id, device=dev)
    out = []
    for i in range(max_new_tokens):
        tok = torch.argmax(logits[..., :vocab], dim=-1)
        tok = torch.where(done, eos, tok)
        done = done | (tok == eos)
        out.append(tok)
        if i < max_new_tokens - 1:
            logits = one_step(tok)
    return torch.stack(out, dim=1)
