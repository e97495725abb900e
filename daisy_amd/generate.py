"""Token generation over a ring KV cache, with the interface of the reference's ``Generator``
(inference/generate.py:61-285): same constructor arguments, ``generate`` is a Python generator
that yields ids and returns ``(history, prefill_seconds, decode_seconds)``, and ``_prefill`` /
``_step`` talk to the model through ``model.prefill(ids[1, T]) -> (logits, kv[2, L, B, H, T, D])``
and ``model.step(token, k_ctxs, v_ctxs, pos) -> (logits, k_list, v_list)``.

What is arranged differently here:

* nothing is wrapped in ``torch.compile``: the hot operations are HIP kernels already;
* when every block's attention is this package's ``CausalSelfAttention`` and the cache is bf16, a
  step hands each layer a handle on its ring (``KVCache.ring``) instead of a chronological copy:
  the decode kernel streams the ring where it lies and appends the new row itself, so a step moves
  no cache bytes on the host's behalf.  The handles are made once, not per token;
* the token history lives in a preallocated buffer that grows geometrically, not in a tensor that
  is re-concatenated for every token.

Sampling follows the reference's arithmetic (inference/generate.py:13-58): temperature, top-k,
nucleus filter, Gumbel-max draw, and the distance-decayed repetition penalty over the last 128
tokens; the random numbers are drawn with the same call, so a seed gives the same tokens.
"""
from __future__ import annotations

import time
from typing import Iterator, List, Optional, Tuple

import torch
from torch import Tensor

from .attention import CausalSelfAttention
from .kv_cache import KVCache

_NEG_INF = float("-inf")
_PENALTY_LOOKBACK = 128      # tokens of history the repetition penalty looks at (generate.py:271)


# ----------------------------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------------------------
def keep_top_k(scores: Tensor, k: Optional[int]) -> Tensor:
    """Everything but the k largest entries of the last dim becomes -inf (no-op for k outside 1..V-1)."""
    vocab = scores.size(-1)
    if not k or k < 0 or k >= vocab:
        return scores
    drop = torch.ones_like(scores, dtype=torch.bool)
    drop.scatter_(-1, scores.topk(k, dim=-1).indices, False)
    return scores.masked_fill(drop, _NEG_INF)


def keep_nucleus(scores: Tensor, p: Optional[float]) -> Tensor:
    """Nucleus filter: in order of falling probability, tokens stay while the running mass is <= p;
    the most likely token always stays (no-op for p outside (0, 1))."""
    if p is None or not (0.0 < p < 1.0):
        return scores
    ranked, order = scores.sort(dim=-1, descending=True)
    mass = ranked.softmax(dim=-1).cumsum(dim=-1)
    out_ranked = mass > p
    out_ranked[..., 0] = False
    out = torch.empty_like(out_ranked).scatter_(-1, order, out_ranked)
    return scores.masked_fill(out, _NEG_INF)


def gumbel_noise(like: Tensor) -> Tensor:
    """Standard Gumbel noise, uniform draw clamped away from 0 at 1e-6."""
    u = torch.rand(like.shape, device=like.device, dtype=like.dtype)
    return u.clamp_min_(1e-6).log_().neg_().log_().neg_()


def sample_token(logits: Tensor, temperature: float = 1.0, top_k: Optional[int] = None,
                 top_p: Optional[float] = None) -> Tensor:
    """Arg-max at temperature 0; otherwise one draw from softmax(filtered logits / temperature)
    by the Gumbel-max identity (arg-max of scores + Gumbel noise)."""
    if temperature == 0.0:
        return logits.argmax(dim=-1)
    scores = keep_nucleus(keep_top_k(logits / max(temperature, 1e-6), top_k), top_p)
    return (scores + gumbel_noise(scores)).argmax(dim=-1)


def penalise_repeats(logits: Tensor, recent: Tensor, strength: Tensor, _one: Optional[Tensor] = None,
                     half_life: float = 140.0, cap: float = 3.0) -> Tensor:
    """A token seen ``d`` positions ago (1 = the last one) counts ``0.5 ** (d / half_life)``; counts
    add up per token and saturate at ``cap``; the token's logit is divided by ``strength ** count``
    when positive and multiplied by it otherwise.  ``_one`` is unused (kept for the call shape).
    Works on one row (``logits [V]``, ``recent [n]``) or on a batch (``[B, V]``, ``[B, n]``)."""
    n = recent.size(-1)
    age = torch.arange(n, 0, -1, device=logits.device, dtype=logits.dtype)
    weight = torch.pow(0.5, age / half_life)
    if logits.dim() == 1:
        count = torch.zeros_like(logits).index_add_(0, recent, weight)
    else:                                   # a batch: logits [B, V], recent [B, n]
        count = torch.zeros_like(logits).scatter_add_(1, recent, weight.expand_as(recent))
    scale = torch.pow(strength, count.clamp_(max=cap))
    return logits * torch.where(logits > 0, scale.reciprocal(), scale)


# ----------------------------------------------------------------------------------------------
# generator
# ----------------------------------------------------------------------------------------------
class Generator:
    def __init__(self, model, window, seed, device=None, dtype=torch.float16, max_seq_len: int = 65536,
                 temperature=1.0, top_k=None, top_p=None, repetition_penalty=1.0, eos_token_id=None,
                 record_steps: bool = False, direct_prefill: bool = False):
        eos = eos_token_id if eos_token_id is not None else getattr(model, "eos_token_id", None)
        if eos is None:
            raise AssertionError("eos_token_id must be given or be an attribute of the model")
        self.model = model.eval()
        self.device = device if device is not None else next(model.parameters()).device
        self.dtype, self.seed, self.max_seq_len = dtype, seed, max_seq_len
        self.temperature, self.top_k, self.top_p = temperature, top_k, top_p
        self.vocab_size = model.embed.num_embeddings
        self.eos_token_id = torch.tensor(eos, device=self.device)
        self.rep_p_t = torch.tensor(repetition_penalty, device=self.device, dtype=dtype)
        self._rep_p_host = float(repetition_penalty)
        self._one = torch.tensor(1, device=self.device, dtype=dtype)
        self.sample = sample_token
        self.apply_repetition_penalty = penalise_repeats

        # Cache geometry comes from the first block that has attention (generate.py:71-76).
        layers = list(model.blocks)
        attn = [getattr(blk, "attn", None) for blk in layers]
        first = next(a for a in attn if a is not None)
        self.cache = KVCache(L=len(layers), B=1, H=first.num_heads, W=window, D=first.head_dim,
                             device=self.device, dtype=dtype)
        # In-place decode: every attention layer must understand ring handles; the ring is bf16, or
        # fp16 (the reference's default, which the decode kernel reads and appends to as it is).
        # (layers that keep their own state, like the KDA layer, never look at their context)
        self.use_ring_context = (dtype in (torch.bfloat16, torch.float16)
                                 and all(a is None or isinstance(a, CausalSelfAttention)
                                         or not getattr(a, "uses_kv_context", True) for a in attn))
        self._rings = [self.cache.ring(i) for i in range(len(layers))] if self.use_ring_context else None
        # record_steps: the decode step is recorded once as a HIP graph and replayed per token
        # (daisy_amd.core.GraphedStep walks the model's layers itself, so the model needs the
        # attributes of the reference's DaisyCore, a bf16 cache and this package's attention).
        self.record_steps = bool(record_steps)
        self._recorded_step = None
        # direct_prefill: the prompt runs through daisy_amd.core.prefill instead of model.prefill: no
        # T x T mask, no [2, L, B, H, T, D] stack, every layer's keys and values go straight into
        # the cache (same requirements on the model as record_steps).
        self.direct_prefill = bool(direct_prefill)
        # generate_batch: one bf16 ring, and one recorded step, per batch size
        self._batch_caches: dict = {}
        self._batch_steps: dict = {}

        torch.manual_seed(seed)
        self._tokens = torch.empty(256, dtype=torch.long, device=self.device)
        self._n_tokens = 0

    # -- history ---------------------------------------------------------------------------
    @property
    def history(self) -> Tensor:
        return self._tokens[:self._n_tokens]

    @history.setter
    def history(self, ids: Tensor) -> None:
        self._n_tokens = 0
        self._remember(ids)

    def _remember(self, ids: Tensor) -> None:
        ids = ids.reshape(-1).to(device=self.device, dtype=torch.long)
        need = self._n_tokens + ids.numel()
        if need > self._tokens.numel():
            grown = torch.empty(max(need, 2 * self._tokens.numel()), dtype=torch.long, device=self.device)
            grown[:self._n_tokens] = self._tokens[:self._n_tokens]
            self._tokens = grown
        self._tokens[self._n_tokens:need] = ids
        self._n_tokens = need

    # -- small setters of the reference's interface ----------------------------------------
    def set_temperature(self, temperature: float):
        self.temperature = float(temperature)
        return self

    def set_repetition_penalty(self, repetition_penalty: float):
        self.rep_p_t = torch.tensor(repetition_penalty, device=self.rep_p_t.device, dtype=self.rep_p_t.dtype)
        self._rep_p_host = float(repetition_penalty)
        return self

    def reset_history(self):
        self.model.reset_history()
        self.cache.reset_history()
        self._n_tokens = 0

    def _sync(self):
        if torch.cuda.is_available() and torch.device(self.device).type == "cuda":
            torch.cuda.synchronize()

    def _trim(self, logits: Tensor) -> Tensor:
        return logits.to(self.dtype)[..., :self.vocab_size]

    def _penalised(self, logits: Tensor, recent: Tensor) -> Tensor:
        """The repetition penalty on ``logits``.  A strength of exactly 1 leaves every logit as it is (``x * 1``,
        ``x / 1``), so the dozen small launches of the stock routine are skipped then; a routine put in its place
        (``apply_repetition_penalty`` is an attribute, as in the reference) is always called."""
        if self._rep_p_host == 1.0 and self.apply_repetition_penalty is penalise_repeats:
            return logits
        return self.apply_repetition_penalty(logits, recent, self.rep_p_t, self._one)

    # -- model calls -----------------------------------------------------------------------
    def _prefill(self, prompt_ids: Tensor) -> Tensor:
        """Runs the prompt, stores its keys and values (the last ``W - 1`` positions fit) and
        returns the logits of its last position, ``[1, vocab]``."""
        n = prompt_ids.numel()
        assert n > 0
        if self.direct_prefill:
            from . import core
            logits, _ = core.prefill(self.model, prompt_ids.view(1, n), self.cache)
        else:
            logits, kv = self.model.prefill(prompt_ids.view(1, n))
            self.cache.bulk_write_packed(kv, n)
        self._remember(prompt_ids)
        return self._trim(logits)

    def _contexts(self) -> Tuple[List, List]:
        if self._rings is not None:
            for ring in self._rings:      # the handles are reused; only the position moves
                ring.t = self.cache.t
            return self._rings, self._rings
        views = [self.cache.view(i) for i in range(self.cache.L)]
        for k, v in views:
            assert k.dtype == self.dtype and v.dtype == self.dtype
        return [k for k, _ in views], [v for _, v in views]

    def _step(self, token: Tensor) -> Tensor:
        """One decode step: the model sees every layer's context as it was before this token,
        the new rows go into slot ``t % W`` (unless the decode kernel has already put them
        there), the cache moves on by one position."""
        if self.record_steps:
            if self._recorded_step is None:
                from . import core
                self._recorded_step = core.GraphedStep(self.model, self.cache)
            logits = self._recorded_step(token)
            self._remember(token)
            return self._trim(logits)
        k_ctxs, v_ctxs = self._contexts()
        logits, k_rows, v_rows = self.model.step(token, k_ctxs, v_ctxs, self.cache.t)
        # A layer without attention returns None; its slot is filled with zeros shaped like the
        # first layer's row, as the reference does (generate.py:240-241).
        blank = None
        for layer, (k_row, v_row) in enumerate(zip(k_rows, v_rows)):
            if self.cache._staged[layer]:
                continue
            if k_row is None or v_row is None:
                if blank is None:
                    # (the reference shapes it like the first layer's row, generate.py:240-241, and so
                    # needs attention in the first layer; the cache's own geometry serves every stack)
                    blank = torch.zeros(self.cache.B, 1, self.cache.H, self.cache.D, device=self.device, dtype=self.dtype)
                k_row = v_row = blank
            self.cache.write(layer, k_row.to(self.dtype), v_row.to(self.dtype))
        self.cache.advance()
        self._remember(token)
        return self._trim(logits)

    # -- the loop --------------------------------------------------------------------------
    @torch.inference_mode()
    def generate(self, prompt_ids: Tensor, max_new_tokens) -> Iterator[Tensor]:
        """Yields one ``[1]`` id tensor per generated token and stops at the end-of-sequence token
        (not yielded) or after ``max_new_tokens``; the generator's return value is
        ``(history, prefill_seconds, decode_seconds)``."""
        assert prompt_ids.ndim == 1 and prompt_ids.numel() > 0 and max_new_tokens > 0
        self.reset_history()
        self._sync()
        t_start = time.perf_counter()
        logits = self._prefill(prompt_ids)
        self._sync()
        t_prompt = time.perf_counter()
        for produced in range(1, max_new_tokens + 1):
            scores = self._penalised(logits[-1], self.history[-_PENALTY_LOOKBACK:])
            token = self.sample(scores, self.temperature, self.top_k, self.top_p)
            if token == self.eos_token_id:
                break
            yield token.view(1)
            if produced < max_new_tokens:
                logits = self._step(token)
            else:
                self._remember(token)     # the last token is recorded but not run through the model
        self._sync()
        t_end = time.perf_counter()
        return self.history.detach().clone(), t_prompt - t_start, t_end - t_prompt

    @torch.inference_mode()
    def generate_batch(self, prompt_ids: Tensor, max_new_tokens: int, record_steps: bool = False) -> Tensor:
        """A batch of equally long prompts ``[B, T]`` -> ``[B, max_new_tokens]`` ids, with the same
        sampling settings as ``generate``.  A row that produces the end-of-sequence token keeps
        emitting it.  The reference's generator is built for one sequence (generate.py:76); this
        path drives the model through ``daisy_amd.core`` (descriptor mask, keys and values of
        every layer written straight into a bf16 ring of batch B, in-place decode steps), so the
        model needs the attributes of the reference's ``DaisyCore`` and this package's attention.

        ``record_steps``: record the decode step once per batch size as a HIP graph
        (``core.GraphedStep``) and replay it for every token instead of launching its kernels
        one by one; the model's parameters must stay where they are between calls.
        """
        from . import core
        assert prompt_ids.ndim == 2 and prompt_ids.size(1) > 0 and max_new_tokens > 0
        ids = prompt_ids.to(self.device)
        B = ids.size(0)
        cache = self._batch_caches.get(B)
        if cache is None:
            cache = self._batch_caches[B] = KVCache(L=self.cache.L, B=B, H=self.cache.H, W=self.cache.W, D=self.cache.D,
                                                    device=self.device, dtype=torch.bfloat16)
        cache.reset_history()
        self.model.reset_history()
        step = lambda tokens: core.step(self.model, tokens, cache)
        if record_steps:
            if B not in self._batch_steps:
                self._batch_steps[B] = core.GraphedStep(self.model, cache)
            step = self._batch_steps[B]
        logits, _ = core.prefill(self.model, ids, cache)
        seen = torch.empty(B, ids.size(1) + max_new_tokens, dtype=torch.long, device=self.device)
        seen[:, :ids.size(1)] = ids
        n_seen = ids.size(1)
        eos = self.eos_token_id.to(torch.long)
        done = torch.zeros(B, dtype=torch.bool, device=self.device)
        for produced in range(1, max_new_tokens + 1):
            scores = self._trim(logits)
            scores = self._penalised(scores, seen[:, max(n_seen - _PENALTY_LOOKBACK, 0):n_seen])
            token = self.sample(scores, self.temperature, self.top_k, self.top_p)
            token = torch.where(done, eos, token)
            done |= token == eos
            seen[:, n_seen] = token
            n_seen += 1
            if produced < max_new_tokens:
                logits = step(token)
        return seen[:, ids.size(1):n_seen].clone()
