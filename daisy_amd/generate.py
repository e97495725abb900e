"""``Generator`` with the reference's interface (inference/generate.py:61-285).

``_prefill`` runs ``model.prefill`` and fills the ring cache, ``_step`` hands the
per-layer context to ``model.step`` and appends the new rows, ``generate``
yields sampled tokens.  Differences from the reference, none visible to a
caller: nothing is wrapped in ``torch.compile`` (the hot ops are HIP kernels),
and when every attention layer is this package's ``CausalSelfAttention`` the
step passes ``RingContext`` handles so the decode kernel streams the cache in
place and appends the new row itself (no chronological copy, no second write).
"""
from __future__ import annotations

import time
from typing import Generator as _GeneratorType

import torch
import torch.nn.functional as F

from .attention import CausalSelfAttention
from .kv_cache import KVCache


def _topk_filter(x, k):
    if k is None or k <= 0 or k >= x.size(-1):
        return x
    vals, idx = torch.topk(x, k)
    return torch.full_like(x, float("-inf")).scatter_(-1, idx, vals)


def _topp_filter(x, p):
    if p is None or p <= 0.0 or p >= 1.0:
        return x
    sorted_p, order = torch.sort(F.softmax(x, dim=-1), dim=-1, descending=True)
    keep_sorted = torch.cumsum(sorted_p, dim=-1) <= p
    keep_sorted[..., 0] = True
    keep = torch.zeros_like(keep_sorted).scatter(-1, order, keep_sorted)
    return x.masked_fill(~keep, float("-inf"))


def _gumbel(shape, device, dtype):
    u = torch.rand(shape, device=device, dtype=dtype)
    return -torch.log(-torch.log(u.clamp_min_(1e-6)))


def _sample(logits, temperature=1.0, top_k=None, top_p=None):
    """Greedy at temperature 0, else Gumbel-max over the filtered logits (generate.py:36-45)."""
    if temperature == 0.0:
        return torch.argmax(logits, dim=-1)
    x = logits / max(temperature, 1e-6)
    x = _topp_filter(_topk_filter(x, top_k), top_p)
    return torch.argmax(x + _gumbel(x.shape, x.device, x.dtype), dim=-1)


def _repetition_penalty(logits, prev: torch.Tensor, rep_p: torch.Tensor, _one: torch.Tensor, rep_h=140.0, cap=3.0):
    """Distance-decayed repetition penalty (generate.py:47-58)."""
    dist = torch.arange(prev.numel(), 0, -1, device=logits.device, dtype=logits.dtype)
    hits = torch.zeros_like(logits).scatter_add_(0, prev, 0.5 ** (dist / rep_h)).clamp_max_(cap)
    scale = torch.pow(rep_p, hits)
    return logits * torch.where(logits > 0, 1.0 / scale, scale)


class Generator:
    def __init__(self, model, window, seed, device=None, dtype=torch.float16, max_seq_len: int = 65536,
                 temperature=1.0, top_k=None, top_p=None, repetition_penalty=1.0, eos_token_id=None):
        if eos_token_id is None:
            eos_token_id = getattr(model, "eos_token_id", None)
        assert eos_token_id is not None
        self.model = model.eval()
        self.device = next(model.parameters()).device if device is None else device
        self.dtype = dtype
        assert self.device is not None
        h = d = None
        attn_modules = []
        for b in self.model.blocks:
            a = getattr(b, "attn", None)
            if a is not None:
                attn_modules.append(a)
                if h is None:
                    h, d = a.num_heads, a.head_dim
        self.cache = KVCache(L=len(self.model.blocks), B=1, H=h, W=window, D=d, device=self.device, dtype=dtype)
        # In-place decode needs every layer's attention to understand RingContext
        # and a bf16 cache (the kernels' storage type).
        self.use_ring_context = (dtype == torch.bfloat16 and len(attn_modules) == len(self.model.blocks)
                                 and all(isinstance(a, CausalSelfAttention) for a in attn_modules))
        self.temperature = temperature
        self.top_k = top_k
        self.top_p = top_p
        self.rep_p_t = torch.tensor(repetition_penalty, device=self.device, dtype=dtype)
        self.eos_token_id = torch.tensor(eos_token_id, device=self.device)
        self.max_seq_len = max_seq_len
        self.vocab_size = self.model.embed.num_embeddings
        self._one = torch.tensor(1, device=self.device, dtype=dtype)
        self.seed = seed
        torch.manual_seed(self.seed)
        self.history = torch.empty(0, dtype=torch.long, device=self.device)
        self.sample = _sample
        self.apply_repetition_penalty = _repetition_penalty

    def _sync(self):
        if str(self.device).startswith("cuda") and torch.cuda.is_available():
            torch.cuda.synchronize()

    def set_temperature(self, temperature: float):
        self.temperature = float(temperature)
        return self

    def set_repetition_penalty(self, repetition_penalty: float):
        self.rep_p_t = torch.tensor(repetition_penalty, device=self.rep_p_t.device, dtype=self.rep_p_t.dtype)
        return self

    def reset_history(self):
        self.model.reset_history()
        self.cache.reset_history()
        self.history = torch.empty(0, dtype=torch.long, device=self.device)

    def _prefill(self, prompt_ids: torch.Tensor):
        """``model.prefill(ids[1, T]) -> (logits, kv[2, L, B, H, T, D])``; fills the cache."""
        ids = prompt_ids[None, :]
        assert ids.size(1) > 0
        logits, kv = self.model.prefill(ids)
        logits = logits.to(self.dtype)[..., :self.vocab_size]
        self.cache.bulk_write_packed(kv, prompt_ids.numel())
        self.history = torch.cat([self.history, prompt_ids.to(dtype=torch.long, device=self.device)], dim=0)
        return logits

    def _step(self, token: torch.Tensor):
        L = len(self.model.blocks)
        k_ctxs, v_ctxs = [], []
        for i in range(L):
            if self.use_ring_context:
                ctx = self.cache.ring(i)
                k_ctxs.append(ctx)
                v_ctxs.append(ctx)
            else:
                kc, vc = self.cache.view(i)
                assert kc.dtype == self.dtype and vc.dtype == self.dtype
                k_ctxs.append(kc)
                v_ctxs.append(vc)
        logits, k_new, v_new = self.model.step(token, k_ctxs, v_ctxs, self.cache.t)
        logits = logits.to(self.dtype)[..., :self.vocab_size]
        # Layers without attention return None; the first layer always has attention.
        k_new = [x.to(self.dtype) if x is not None else torch.zeros_like(k_new[0]) for x in k_new]
        v_new = [x.to(self.dtype) if x is not None else torch.zeros_like(v_new[0]) for x in v_new]
        for i in range(L):
            if not self.cache._staged[i]:  # the decode kernel may already have appended this row
                self.cache.write(i, k_new[i], v_new[i])
        self.cache.advance()
        self.history = torch.cat([self.history, token.view(1)], dim=0)
        return logits

    @torch.inference_mode()
    def generate(self, prompt_ids: torch.Tensor, max_new_tokens) -> _GeneratorType[torch.Tensor, None, tuple]:
        """Yields generated ids; returns ``(history, prefill_seconds, step_seconds)``."""
        assert prompt_ids.ndim == 1
        assert prompt_ids.size(0) > 0
        assert max_new_tokens > 0
        self.reset_history()
        self._sync(); t0 = time.perf_counter()
        logits = self._prefill(prompt_ids)
        self._sync(); t1 = time.perf_counter()
        for i in range(max_new_tokens):
            logits = logits[-1]
            prev_ids = self.history[-128:]
            logits = self.apply_repetition_penalty(logits, prev_ids, self.rep_p_t, self._one)
            tok = self.sample(logits, self.temperature, self.top_k, self.top_p)
            if tok == self.eos_token_id:
                break
            yield tok.view(1)
            if i < max_new_tokens - 1:
                logits = self._step(tok)
            else:
                t = tok.to(device=self.device, dtype=torch.long).reshape(())
                self.history = torch.cat([self.history, t.view(1)], dim=0)
                logits = None
        self._sync(); t2 = time.perf_counter()
        return self.history.detach().clone(), t1 - t0, t2 - t1
