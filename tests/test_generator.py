"""Generator plumbing with a one-hot fake model: the scenarios of the
reference's tests/test_generator.py:128-189,251-277 (prefill fills the cache in
order, step passes pre-write contexts and appends, greedy generation)."""
import pytest
import torch
import torch.nn as nn

from daisy_amd import Generator


class FakeAttn:
    def __init__(self, num_heads, head_dim):
        self.num_heads, self.head_dim = num_heads, head_dim


class FakeBlock(nn.Module):
    def __init__(self, attn):
        super().__init__()
        self.attn = attn


class OneHotModel(nn.Module):
    """embed = identity, logits = embedding of the current token, K = V = embedding."""

    def __init__(self, vocab, layers=2):
        super().__init__()
        self.eos_token_id = 50256
        self.embed = nn.Embedding(vocab, vocab)
        with torch.no_grad():
            self.embed.weight.copy_(torch.eye(vocab))
        self.blocks = nn.ModuleList([FakeBlock(FakeAttn(1, vocab)) for _ in range(layers)])
        self.seen_k = self.seen_v = None

    def reset_history(self):
        self.seen_k = self.seen_v = None

    @torch.no_grad()
    def prefill(self, ids):
        B, T = ids.shape
        e = self.embed(ids)
        k = e.view(B, T, 1, -1).transpose(1, 2)
        K = torch.stack([k for _ in self.blocks])
        return e[:, -1], torch.stack([K, K.clone()])

    @torch.no_grad()
    def step(self, token_id, k_ctxs, v_ctxs, pos):
        self.seen_k = [k.clone() for k in k_ctxs]
        self.seen_v = [v.clone() for v in v_ctxs]
        e = self.embed(token_id)
        kv = e.view(1, 1, 1, -1)
        return e.view(1, -1), [kv for _ in self.blocks], [kv.clone() for _ in self.blocks]


V = 16


DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


@pytest.fixture(params=DEVICES)
def env(request):
    """(model, generator, device): the scenarios run on CPU tensors and, under the ``gpu`` mark, with model,
    cache and prompts on ``cuda:0``, where the generator is used."""
    torch.manual_seed(0)
    dev = torch.device(request.param)
    model = OneHotModel(V).to(dev).eval()
    gen = Generator(model, window=8, seed=1337, device=dev, dtype=torch.bfloat16, temperature=0.0)
    return model, gen, dev


def onehot(i):
    v = torch.zeros(V)
    v[i] = 1.0
    return v


def eq(got, want):
    return torch.equal(got.float().cpu(), want.float().cpu())


def test_prefill_updates_cache_and_returns_logits(env):
    model, gen, dev = env
    prompt = torch.tensor([3, 5, 7, 9], device=dev)
    logits = gen._prefill(prompt)
    assert logits.shape == (1, V) and eq(logits[0], onehot(9))
    assert gen.cache.t == 4
    for layer in range(2):
        k, v = gen.cache.view(layer)
        assert k.shape == (1, 4, 1, V)
        for t, tok in enumerate(prompt.tolist()):
            assert eq(k[0, t, 0], onehot(tok)) and eq(v[0, t, 0], onehot(tok))
    assert torch.equal(gen.history, prompt) and gen.cache.k.device == dev and logits.device == dev
    assert gen.use_ring_context is False   # a foreign model gets chronological tensors


def test_step_writes_kv_and_advances_cache(env):
    model, gen, dev = env
    gen._prefill(torch.tensor([2, 4, 6], device=dev))
    t0 = gen.cache.t
    logits = gen._step(torch.tensor(11, device=dev))
    assert eq(logits[0], onehot(11))
    assert gen.cache.t == t0 + 1
    for layer in range(2):
        k, v = gen.cache.view(layer)
        assert eq(k[0, -1, 0], onehot(11)) and eq(v[0, -1, 0], onehot(11))
        # the model saw the cache as it was BEFORE this token's row was written
        assert eq(model.seen_k[layer], k[:, :-1])
        assert eq(model.seen_v[layer], v[:, :-1])
    assert gen.history[-1].item() == 11


def test_window_limits_what_prefill_stores(env):
    model, gen, dev = env
    prompt = torch.arange(12, device=dev) % V
    gen._prefill(prompt)
    k, _ = gen.cache.view(0)          # W = 8: a view shows 8 rows, bulk write stored the last W - 1 = 7
    assert k.shape[1] == 8
    for j, tok in enumerate(prompt[-7:].tolist()):
        assert eq(k[0, 1 + j, 0], onehot(tok))


def test_generate_end_to_end(env):
    model, gen, dev = env
    prompt = torch.tensor([4, 1, 4], device=dev)
    assert [int(t) for t in gen.generate(prompt, max_new_tokens=3)] == [4, 4, 4]
    g = gen.generate(prompt, max_new_tokens=2)
    toks = []
    try:
        while True:
            toks.append(int(next(g)))
    except StopIteration as e:
        out, pre, step = e.value
    assert toks == [4, 4] and out.tolist() == [4, 1, 4, 4, 4]
    assert isinstance(pre, float) and isinstance(step, float)


def test_sampling_helpers():
    model = OneHotModel(8, layers=1)
    gen = Generator(model, window=4, seed=1, device=torch.device("cpu"), dtype=torch.bfloat16)
    gen.history = torch.tensor([1, 2, 3, 2, 1])
    logits = torch.tensor([0.1, 0.9, 0.5, -1.0, 0.0, 0.0, 0.0, 0.0])
    assert int(gen.sample(logits, 0.0, None, None)) == 1
    assert int(gen.sample(logits, 1.0, 1, None)) == 1                 # top-1 == argmax
    assert 0 <= int(gen.sample(logits, 1.0, None, 0.6)) <= 2           # nucleus keeps {1, 2, 0}
    gen.set_repetition_penalty(1.2)
    l2 = torch.tensor([0.95, 0.94, 0.93, 0.0, 0.0, 0.0, 0.0, 0.0])
    pen = gen.apply_repetition_penalty(l2, gen.history[-128:], gen.rep_p_t.float(), gen._one)
    assert int(torch.argmax(pen)) == 0                                   # tokens 1 and 2 were seen, 0 was not


def test_a_penalty_of_one_is_the_identity_and_skipped():
    """A repetition penalty of exactly 1 changes no logit (inference/generate.py:47-58: scale = 1 ** count), so the
    generator does not launch the routine for it -- unless a caller has put a routine of their own in its place."""
    from daisy_amd.generate import penalise_repeats
    model = OneHotModel(8, layers=1)
    gen = Generator(model, window=4, seed=1, device=torch.device("cpu"), dtype=torch.bfloat16)
    recent = torch.tensor([1, 2, 3, 2, 1])
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        logits = torch.tensor([0.1, -0.9, 0.5, -1.0, 3.0, 0.0, -7.5, 2.25], dtype=dt)
        assert torch.equal(penalise_repeats(logits, recent, torch.tensor(1.0, dtype=dt)), logits)
        assert gen._penalised(logits, recent) is logits
    calls = []
    gen.apply_repetition_penalty = lambda lg, prev, strength, one: (calls.append(float(strength)), lg + 1)[1]
    out = gen._penalised(torch.zeros(8), recent)
    assert calls == [1.0] and torch.equal(out, torch.ones(8))
    gen.apply_repetition_penalty = penalise_repeats
    gen.set_repetition_penalty(1.3)
    want = penalise_repeats(torch.ones(8, dtype=torch.bfloat16), recent, gen.rep_p_t, gen._one)
    assert torch.equal(gen._penalised(torch.ones(8, dtype=torch.bfloat16), recent), want) and not torch.equal(want, torch.ones(8, dtype=torch.bfloat16))
    gen.set_repetition_penalty(1.0)
    assert gen._penalised(want, recent) is want
