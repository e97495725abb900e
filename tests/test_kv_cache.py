"""KV-cache semantics: the reference's known-answer scenarios (kept as data in
tests/golden/kv_cache_scenarios.json) against BOTH the oracle ring buffer and
the product ``daisy_amd.KVCache`` -- on CPU tensors (the cache is host bookkeeping
around torch indexing) and, under the ``gpu`` mark, on ``cuda:0`` tensors, where the
generator keeps it."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from daisy_amd import KVCache

with open(os.path.join(os.path.dirname(__file__), "golden", "kv_cache_scenarios.json")) as f:
    GOLD = json.load(f)


KINDS = ["oracle", "product", pytest.param("product_gpu", marks=pytest.mark.gpu)]
PRODUCT_KINDS = ["product", pytest.param("product_gpu", marks=pytest.mark.gpu)]


def _device(kind):
    return "cuda:0" if kind == "product_gpu" else "cpu"


def _make(kind, L, B, H, W, D, dtype=torch.float32):
    if kind == "oracle":
        return oracle.RingKVCache(L, B, H, W, D)
    return KVCache(L=L, B=B, H=H, W=W, D=D, device=_device(kind), dtype=dtype)


def _arg(kind, t, as_float=False):
    """A tensor as the cache of this kind takes it: numpy for the oracle, on the cache's device for the product."""
    if kind == "oracle":
        return (t.float() if as_float else t).numpy()
    return t.to(_device(kind))


def _np(x):
    return x.float().cpu().numpy() if isinstance(x, torch.Tensor) else np.asarray(x)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("sc", GOLD["scenarios"], ids=lambda s: s["name"])
def test_scenarios(kind, sc):
    L, B, H, W, D = (sc[k] for k in "LBHWD")
    cache = _make(kind, L, B, H, W, D)
    for val in sc["writes"]:
        k_new = torch.full((B, H, 1, D), val)
        v_new = torch.full((B, H, 1, D), val + 1000.0)
        cache.write(0, _arg(kind, k_new), _arg(kind, v_new))
        cache.advance()
    k, v = cache.view(sc["view_layer"])
    n = len(sc["expect"])
    assert tuple(k.shape) == (B, n, H, D) and tuple(v.shape) == (B, n, H, D)
    for j, val in enumerate(sc["expect"]):
        assert (_np(k)[:, j] == val).all() and (_np(v)[:, j] == val + 1000.0).all()
    assert cache.t == len(sc["writes"])


@pytest.mark.parametrize("kind", KINDS)
def test_write_accepts_B_1_H_D(kind):
    L, B, H, W, D = 1, 2, 3, 2, 4
    cache = _make(kind, L, B, H, W, D)
    k_new, v_new = torch.randn(B, 1, H, D), torch.randn(B, 1, H, D)
    cache.write(0, _arg(kind, k_new), _arg(kind, v_new))
    cache.advance()
    k, v = cache.view(0)
    assert np.array_equal(_np(k), k_new.numpy()) and np.array_equal(_np(v), v_new.numpy())
    assert kind == "oracle" or (k.device == torch.device(_device(kind)) and cache.k.device == k.device)


@pytest.mark.parametrize("kind", KINDS)
def test_reset(kind):
    cache = _make(kind, 1, 2, 2, 3, 2)
    for i in range(2):
        kn = torch.full((2, 2, 1, 2), 30.0 + i)
        cache.write(0, _arg(kind, kn), _arg(kind, kn))
        cache.advance()
    cache.reset_history()
    assert cache.t == 0
    k, v = cache.view(0)
    assert tuple(k.shape) == (2, 0, 2, 2)
    assert float(np.abs(_np(cache.k)).sum()) == 0.0


@pytest.mark.parametrize("kind", KINDS)
def test_staged_write_visibility_and_contract(kind):
    g = GOLD["staged_view"]
    W, steps, L, B, H, D = (g[k] for k in ("W", "steps", "L", "B", "H", "D"))
    cache = _make(kind, L, B, H, W, D, dtype=torch.bfloat16)
    for t in range(steps):
        for layer in range(L):
            k_ctx, _ = cache.view(layer)
            assert k_ctx.shape[1] == min(t, W)                       # before the write: min(t, W) rows
        kn = torch.full((B, H, 1, D), float(t), dtype=torch.bfloat16)
        for layer in range(L):
            cache.write(layer, _arg(kind, kn, True), _arg(kind, kn, True))
        for layer in range(L):
            k_ctx, _ = cache.view(layer)                               # staged: min(t + 1, W) rows, newest last
            got = [int(x) for x in _np(k_ctx)[0, :, 0, 0]]
            n = min(t + 1, W)
            assert got == list(range(t - n + 1, t + 1))
        cache.advance()


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("sc", GOLD["bulk"], ids=lambda s: f"W{s['W']}_T{s['T']}")
def test_bulk_write_packed(kind, sc):
    L, B, H, D, W, T = 2, 1, 2, 3, sc["W"], sc["T"]
    cache = _make(kind, L, B, H, W, D)
    pos = torch.arange(T, dtype=torch.float32)
    kv = pos.view(1, 1, 1, 1, T, 1).expand(2, L, B, H, T, D).clone()
    kv[1] += 1000.0
    cache.bulk_write_packed(_arg(kind, kv), T)
    assert cache.t == sc["expect_t"]
    for layer in range(L):
        k, v = cache.view(layer)
        # view() exposes min(t, W) rows; of those only the last min(T, W - 1) were stored by the bulk write
        n_stored = len(sc["expect_view"])
        got_k = [int(x) for x in _np(k)[0, :, 0, 0]][-n_stored:] if n_stored else []
        got_v = [int(x) for x in _np(v)[0, :, 0, 0]][-n_stored:] if n_stored else []
        assert got_k == sc["expect_view"]
        assert got_v == [x + 1000 for x in sc["expect_view"]]


@pytest.mark.parametrize("kind", PRODUCT_KINDS)
def test_product_matches_oracle_on_random_traffic(kind):
    """Random interleaving of bulk writes, staged writes and advances: identical views."""
    rng = np.random.default_rng(0)
    L, B, H, W, D = 2, 2, 2, 5, 3
    a, b = _make("oracle", L, B, H, W, D), _make(kind, L, B, H, W, D)
    dev = _device(kind)
    T0 = 7
    kv = rng.standard_normal((2, L, B, H, T0, D)).astype(np.float32)
    a.bulk_write_packed(kv, T0)
    b.bulk_write_packed(torch.from_numpy(kv).to(dev), T0)
    for step in range(13):
        for layer in range(L):
            kn = rng.standard_normal((B, 1, H, D)).astype(np.float32)
            vn = rng.standard_normal((B, 1, H, D)).astype(np.float32)
            a.write(layer, kn, vn)
            b.write(layer, torch.from_numpy(kn).to(dev), torch.from_numpy(vn).to(dev))
            ka, va = a.view(layer)
            kb, vb = b.view(layer)
            # the slot skipped by the bulk write is visible but unspecified for the first steps: compare stored rows
            lo = max(0, ka.shape[1] - (min(T0, W - 1) + step + 1))
            assert np.array_equal(ka[:, lo:], _np(kb)[:, lo:]) and np.array_equal(va[:, lo:], _np(vb)[:, lo:])
        a.advance(); b.advance()
    assert a.t == b.t == T0 + 13


@pytest.mark.parametrize("kind", PRODUCT_KINDS)
def test_ring_context_is_a_view(kind):
    cache = KVCache(L=2, B=1, H=2, W=4, D=8, device=_device(kind), dtype=torch.bfloat16)
    ring = cache.ring(1)
    assert ring.k.data_ptr() == cache.k[1].data_ptr() and ring.W == 4 and ring.t == 0
    ring.mark_written()
    assert cache._staged == [False, True]


def test_bf16_rows_survive_an_fp16_cache():
    """The reference's generator keeps its cache in fp16 by default (inference/generate.py:62) while the
    model's keys and values are bf16.  bf16 has fewer mantissa bits than fp16, so the conversion loses
    nothing inside fp16's normal range (|x| >= 2^-14; normalised rows never exceed sqrt(D)); below it
    the absolute error stays under 2^-25.  The decode kernel relies on this when it appends to and
    reads from an fp16 ring."""
    import torch
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4096, 128, generator=g)
    rows = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    back = rows.half().bfloat16()
    normal = rows.float().abs() >= 2.0 ** -14
    assert torch.equal(back[normal], rows[normal])
    assert (back.float() - rows.float()).abs().max().item() <= 2.0 ** -25
    assert rows.float().abs().max().item() <= 128 ** 0.5 + 0.1
    # and a ring written through fp16 reads back what a bf16 ring holds
    from daisy_amd import KVCache
    a = KVCache(1, 2, 2, 8, 16, "cpu", torch.bfloat16)
    b = KVCache(1, 2, 2, 8, 16, "cpu", torch.float16)
    for t in range(11):
        k, v = (torch.randn(2, 1, 2, 16, generator=g).bfloat16() for _ in range(2))
        for c in (a, b):
            c.write(0, k.to(c.dtype), v.to(c.dtype))
            c.advance()
    ka, va = a.view(0)
    kb, vb = b.view(0)
    assert torch.equal(ka.float(), kb.float()) and torch.equal(va.float(), vb.float())
