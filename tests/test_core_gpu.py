"""Cache-aware prefill / step glue (daisy_amd.core) on a small Daisy-shaped model.

The model below has the attributes of the reference's DaisyCore (models/daisy/daisy_core.py:96-175)
and blocks with the arithmetic of models/daisy/block.py:33-81.  Checked: against an fp32-softmax CPU
evaluation of the same model through the oracle's attention; that writing K/V straight into the ring
equals the reference's stack-then-bulk_write_packed route bit for bit; that steps through the ring match
steps over chronological views; and that a batch of sequences gives what each sequence gives alone.
"""
import os

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

os.environ["DISABLE_O_ZERO_INIT"] = "1"

import oracle
from daisy_amd import CausalSelfAttention, KVCache, core
from daisy_amd.functional import norm
from helpers import say

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class _MLP(nn.Module):
    def __init__(self, dim):
        super().__init__()
        self.fc = nn.Parameter((torch.randn(2 * dim, dim) * 0.05).bfloat16())
        self.proj = nn.Parameter((torch.randn(dim, 2 * dim) * 0.05).bfloat16())

    def forward(self, x):
        return F.linear(F.relu(F.linear(x, self.fc)).square(), self.proj)


class _Block(nn.Module):
    def __init__(self, dim, H, D, has_attn, receives_ve, max_seq_len):
        super().__init__()
        self.g_x = nn.Parameter(torch.tensor(2.0))
        self.attn = CausalSelfAttention(dim, H, D, receives_ve=receives_ve, max_seq_len=max_seq_len) if has_attn else None
        if self.attn is not None:
            with torch.no_grad():
                self.attn.qkvo_w.copy_((torch.randn(4, dim, dim) * 0.04).bfloat16())
        self.mlp = _MLP(dim)

    def _mix(self, x, x0):
        g = torch.sigmoid(self.g_x)
        return g * x + (1.0 - g) * x0

    def prefill(self, x, ve, x0, attn_mask=None, debug=False):
        x = self._mix(x, x0)
        k = v = None
        if self.attn is not None:
            y, k, v = self.attn.prefill(x, ve, attn_mask, debug=debug)
            x = x + y
        return x + self.mlp(norm(x)), k, v

    def step(self, x, ve, x0, k_ctx, v_ctx, pos, window):
        x = self._mix(x, x0)
        k = v = None
        if self.attn is not None:
            y, k, v = self.attn.step(x, k_ctx, v_ctx, pos, ve, window=window)
            x = x + y
        return x + self.mlp(norm(x)), k, v


class _Core(nn.Module):
    """L = 4 layers, attention in layers 0, 1, 3 (layer 2 has none), value embeddings into 0 and 3, skip 1 -> 3."""

    def __init__(self, vocab=96, dim=256, H=2, D=128, window=48, eos=1, max_seq_len=512):
        super().__init__()
        torch.manual_seed(0)
        self.embed = nn.Embedding(vocab, dim)
        self.attn_layers = [0, 1, 3]
        self.blocks = nn.ModuleList([_Block(dim, H, D, i in self.attn_layers, i in (0, 3), max_seq_len) for i in range(4)])
        self.ve_emb = nn.Embedding(vocab, dim)
        self.ve_module_map = {0: self.ve_emb, 3: self.ve_emb}
        self.skip_map = {3: 1}
        self.skip_weights = nn.Parameter(torch.ones(4) * 1.5)
        self.lm_head_w = nn.Parameter(torch.randn(128, dim) * 0.05)
        self.window_size = self.attn_window_size = window
        self.eos_token_id = eos
        self.attn_num_heads, self.attn_head_dim = H, D
        self.bfloat16()

    def compute_value_embeddings(self, ids):
        return {i: m(ids) for i, m in self.ve_module_map.items()}

    def prefill(self, ids):        # the reference's signature: logits of the last position and kv [2, L, B, H, T, D]
        return core.prefill(self, ids)

    def reset_history(self):
        for blk in self.blocks:
            if blk.attn is not None:
                blk.attn.reset_history()

    # the reference's own step signature (daisy_core.py:294-323), used as the comparison route
    def step(self, token_id, k_ctxs, v_ctxs, pos):
        token_id = token_id.view(1, 1)
        x = x0 = norm(self.embed(token_id))
        ve_map = self.compute_value_embeddings(token_id)
        skips, ks, vs = [], [], []
        for i, blk in enumerate(self.blocks):
            if i in self.skip_map:
                gate = torch.sigmoid(self.skip_weights[self.skip_map[i]])
                x = x * gate + (1 - gate) * skips[self.skip_map[i]]
            x, k, v = blk.step(x, ve_map.get(i), x0, k_ctxs[i], v_ctxs[i], pos, self.attn_window_size)
            skips.append(x)
            ks.append(k)
            vs.append(v)
        return F.linear(norm(x).flatten(end_dim=1).bfloat16(), self.lm_head_w.bfloat16()).float(), ks, vs


def _cpu_prefill_logits(model_cpu, ids):
    """The same model evaluated on the CPU with the oracle's attention (fp32 softmax and contractions)."""
    m = model_cpu
    T = ids.size(1)
    x = x0 = oracle.rms_norm(m.embed(ids))
    ve_map = m.compute_value_embeddings(ids)
    doc_start = oracle.doc_start_from_ids(ids, m.eos_token_id)
    skips = []
    for i, blk in enumerate(m.blocks):
        if i in m.skip_map:
            gate = torch.sigmoid(m.skip_weights[m.skip_map[i]])
            x = x * gate + (1 - gate) * skips[m.skip_map[i]]
        x = blk._mix(x, x0)
        if blk.attn is not None:
            a = blk.attn
            ve = ve_map.get(i)
            y, _, _ = oracle.attn_prefill(x, a.qkvo_w.detach(), a.num_heads, a.head_dim, a.rotary.cos[:T], a.rotary.sin[:T],
                                          m.window_size, doc_start=doc_start, ve=ve,
                                          g_ve=None if a.g_ve is None else float(a.g_ve))
            x = x + y
        x = x + blk.mlp(oracle.rms_norm(x))
        skips.append(x)
    return F.linear(oracle.rms_norm(x)[:, -1].bfloat16(), m.lm_head_w.bfloat16()).float()


def _close(a, b, what, tol=3e-2):
    err = (a.float().cpu() - b.float().cpu()).abs().max().item()
    ref = b.float().abs().max().item()
    say(f"{what}: max-abs diff {err:.3e} (scale {ref:.2f})")
    assert err <= tol * max(ref, 1.0), f"{what}: {err:.3e}"


def test_prefill_matches_cpu_model_and_fills_the_ring_like_the_reference_route():
    with torch.no_grad():
        model_cpu = _Core()
        model = _Core().to(DEV)
        model.load_state_dict(model_cpu.state_dict())
        T, W = 150, model.window_size
        ids = torch.randint(2, 96, (1, T), generator=torch.Generator().manual_seed(3))
        ids[0, 40] = ids[0, 97] = model.eos_token_id          # three documents
        logits_ref = _cpu_prefill_logits(model_cpu, ids)
        logits, kv = core.prefill(model, ids.to(DEV))           # reference-style return value
        assert kv.shape == (2, 4, 1, 2, T, 128)
        assert torch.count_nonzero(kv[:, 2]) == 0              # the layer without attention packs zeros
        _close(logits, logits_ref, "prefill logits vs CPU model")
        # straight into the ring == stack + bulk_write_packed (inference/kv_cache.py:57-68)
        c_ref = KVCache(4, 1, 2, W, 128, DEV, torch.bfloat16)
        c_ref.bulk_write_packed(kv, T)
        c_new = KVCache(4, 1, 2, W, 128, DEV, torch.bfloat16)
        logits2, none = core.prefill(model, ids.to(DEV), c_new)
        assert none is None and c_new.t == T == c_ref.t
        assert torch.equal(logits2, logits)
        assert torch.equal(c_new.k, c_ref.k) and torch.equal(c_new.v, c_ref.v)


def test_steps_through_the_ring_match_steps_over_chronological_views():
    with torch.no_grad():
        model = _Core().to(DEV)
        T, n_steps, W = 70, 60, model.window_size                  # the ring wraps during the steps
        ids = torch.randint(2, 96, (1, T + n_steps), generator=torch.Generator().manual_seed(4)).to(DEV)
        ring = KVCache(4, 1, 2, W, 128, DEV, torch.bfloat16)
        chrono = KVCache(4, 1, 2, W, 128, DEV, torch.bfloat16)
        core.prefill(model, ids[:, :T], ring)
        core.prefill(model, ids[:, :T], chrono)
        for s in range(n_steps):
            tok = ids[0, T + s]
            la = core.step(model, tok, ring)
            views = [chrono.view(i) for i in range(4)]
            lb, ks, vs = model.step(tok, [v[0] for v in views], [v[1] for v in views], chrono.t)
            for i in range(4):
                if ks[i] is not None:
                    chrono.write(i, ks[i], vs[i])
            chrono.advance()
            _close(la, lb, f"step {s} logits", tol=2e-2)
        assert ring.t == chrono.t == T + n_steps
        # same rows in the same slots; the attention-less layer's slots stay zero in both
        _close(ring.k, chrono.k, "ring keys", tol=2e-2)
        _close(ring.v, chrono.v, "ring values", tol=2e-2)
        assert torch.count_nonzero(ring.k[2]) == 0


def test_batched_prefill_and_steps_match_single_sequences():
    with torch.no_grad():
        model = _Core().to(DEV)
        B, T, n_steps, W = 3, 64, 8, model.window_size
        ids = torch.randint(2, 96, (B, T + n_steps), generator=torch.Generator().manual_seed(5)).to(DEV)
        cache = KVCache(4, B, 2, W, 128, DEV, torch.bfloat16)
        lb = [core.prefill(model, ids[:, :T], cache)[0]]
        for s in range(n_steps):
            lb.append(core.step(model, ids[:, T + s], cache))
        for b in range(B):
            c1 = KVCache(4, 1, 2, W, 128, DEV, torch.bfloat16)
            l1 = [core.prefill(model, ids[b:b + 1, :T], c1)[0]]
            for s in range(n_steps):
                l1.append(core.step(model, ids[b, T + s], c1))
            for s in range(n_steps + 1):
                _close(lb[s][b:b + 1], l1[s], f"row {b} call {s}", tol=2e-2)
            _close(cache.k[:, b:b + 1], c1.k, f"row {b} ring keys", tol=2e-2)
        out = core.generate_greedy(model, ids[:, :T], 6)
        assert out.shape == (B, 6) and out.dtype == torch.long
        assert torch.equal(core.generate_greedy(model, ids[:, :T], 6, record_steps=True), out)
        with pytest.raises(Exception, match="end-of-sequence"):
            bad = ids[:, :T].clone()
            bad[1, 5] = model.eos_token_id
            core.prefill(model, bad, KVCache(4, B, 2, W, 128, DEV, torch.bfloat16))


@pytest.mark.parametrize("window,T,n_steps", [(48, 20, 60), (1024, 1000, 40)])
def test_recorded_step_replays_match_eager_steps(window, T, n_steps):
    """core.GraphedStep: the step is recorded once and replayed with the position in device memory.
    Every replay is checked against an eager step on a second cache, with eager work and a
    synchronisation between replays; the ring is partly filled at first and wraps during the run
    (the 1024-slot ring is read by several splits per head).  A cache that is reset and filled
    again keeps working with the same recording."""
    with torch.no_grad():
        model = _Core(window=window, max_seq_len=2048).to(DEV)
        B = 2
        ids = torch.randint(2, 96, (B, T + n_steps), generator=torch.Generator().manual_seed(8)).to(DEV)
        eager = KVCache(4, B, 2, window, 128, DEV, torch.bfloat16)
        replayed = KVCache(4, B, 2, window, 128, DEV, torch.bfloat16)
        core.prefill(model, ids[:, :T], eager)
        core.prefill(model, ids[:, :T], replayed)
        graphed = core.GraphedStep(model, replayed)
        worst = 0.0
        for s in range(n_steps):
            say(f"recorded step W{window} replay {s}")
            want = core.step(model, ids[:, T + s], eager)
            got = graphed(ids[:, T + s]).clone()
            torch.cuda.synchronize()
            worst = max(worst, (got - want).abs().max().item())
            _close(got, want, f"replay {s} logits", tol=1e-2)
        say(f"recorded step W{window}: worst logit difference over {n_steps} replays {worst:.3e}")
        assert replayed.t == eager.t == T + n_steps and int(graphed.pos) == replayed.t
        _close(replayed.k, eager.k, "ring keys", tol=1e-2)
        _close(replayed.v, eager.v, "ring values", tol=1e-2)
        # a new prompt in the same cache: the recording follows the cache's position
        for c in (eager, replayed):
            c.reset_history()
            core.prefill(model, ids[:, 3:T], c)
        for s in range(3):
            want = core.step(model, ids[:, T + s], eager)
            _close(graphed(ids[:, T + s]), want, f"after reset, replay {s} logits", tol=1e-2)
        # the walk cannot be recorded over chronological views
        with pytest.raises(Exception):
            core.GraphedStep(model, KVCache(4, B, 2, window, 128, DEV, torch.float32))


def test_recorded_step_with_a_kda_layer():
    """A hybrid stack (KDA layer first, attention layers after it): the KDA layer keeps its recurrent
    state and convolution windows in buffers whose addresses survive reset_history, so the recording
    made for the first prompt also serves the second one."""
    import copy
    from daisy_amd import KimiLinearSelfAttention
    with torch.no_grad():
        model = _Core(window=48, max_seq_len=512)
        torch.manual_seed(1)
        model.blocks[0].attn = KimiLinearSelfAttention(256, 2, 512, 128, receives_ve=True).bfloat16()
        model = model.to(DEV)
        twin = copy.deepcopy(model)
        B, T, n_steps = 2, 30, 40
        ids = torch.randint(2, 96, (B, T + n_steps), generator=torch.Generator().manual_seed(9)).to(DEV)
        eager = KVCache(4, B, 2, 48, 128, DEV, torch.bfloat16)
        replayed = KVCache(4, B, 2, 48, 128, DEV, torch.bfloat16)
        graphed = None
        for first in (0, 5):                                  # two prompts, one recording
            for m, c in ((model, eager), (twin, replayed)):
                for blk in m.blocks:
                    if blk.attn is not None:
                        blk.attn.reset_history()
                c.reset_history()
                core.prefill(m, ids[:, first:T], c)
            if graphed is None:
                graphed = core.GraphedStep(twin, replayed)
            for s in range(n_steps):
                say(f"recorded hybrid step, prompt from {first}, replay {s}")
                want = core.step(model, ids[:, T + s], eager)
                got = graphed(ids[:, T + s])
                _close(got, want, f"prompt from {first}, replay {s} logits", tol=1e-2)
            _close(twin.blocks[0].attn._recurrent_state, model.blocks[0].attn._recurrent_state, "KDA state", tol=1e-2)
            _close(replayed.k, eager.k, "ring keys", tol=1e-2)
        # the one-sequence generator on the hybrid stack: rings for the attention layers, recorded steps
        from daisy_amd import Generator
        kw = dict(window=48, seed=5, device=torch.device(DEV), dtype=torch.bfloat16, temperature=0.0)
        plain, recorded = Generator(model, **kw), Generator(twin, record_steps=True, direct_prefill=True, **kw)
        assert plain.use_ring_context
        want = torch.cat(list(plain.generate(ids[0, :T], 20)))
        got = torch.cat(list(recorded.generate(ids[0, :T], 20)))
        say(f"hybrid generator: {want.tolist()} vs {got.tolist()}")
        assert torch.equal(want, got)


def test_recorded_step_follows_a_weight_that_changes_in_place():
    """The KDA layer's decode step reads a stacked snapshot of six of its weights; a recording made before one of
    them changed in place (a state dict loaded into the same model) must not go on replaying the old snapshot."""
    import copy
    from daisy_amd import KimiLinearSelfAttention
    with torch.no_grad():
        model = _Core(window=48, max_seq_len=512)
        torch.manual_seed(2)
        model.blocks[0].attn = KimiLinearSelfAttention(256, 2, 512, 128).bfloat16()
        model = model.to(DEV)
        twin = copy.deepcopy(model)
        B, T = 1, 20
        ids = torch.randint(2, 96, (B, T + 12), generator=torch.Generator().manual_seed(4)).to(DEV)
        eager = KVCache(4, B, 2, 48, 128, DEV, torch.bfloat16)
        replayed = KVCache(4, B, 2, 48, 128, DEV, torch.bfloat16)
        core.prefill(model, ids[:, :T], eager)
        core.prefill(twin, ids[:, :T], replayed)
        graphed = core.GraphedStep(twin, replayed)
        for s in range(4):
            _close(graphed(ids[:, T + s]), core.step(model, ids[:, T + s], eager), f"replay {s}", tol=1e-2)
        first_graph = graphed._graph
        for m in (model, twin):                      # the same in-place change on both
            m.blocks[0].attn.v_proj.weight.mul_(-1.0)
        for s in range(4, 8):
            _close(graphed(ids[:, T + s]), core.step(model, ids[:, T + s], eager), f"replay {s} after the change", tol=1e-2)
        assert graphed._graph is not first_graph, "the step was recorded again"


def test_generator_single_sequence_with_recorded_steps():
    """Generator.generate (the reference's one-sequence loop) with record_steps and direct_prefill: the
    same tokens as through model.prefill + bulk_write_packed and steps launched kernel by kernel, for
    two prompts in a row on one generator (one recording)."""
    from daisy_amd import Generator
    with torch.no_grad():
        model = _Core().to(DEV)
        kw = dict(window=model.window_size, seed=3, device=torch.device(DEV), dtype=torch.bfloat16, temperature=0.0)
        plain, recorded = Generator(model, **kw), Generator(model, record_steps=True, direct_prefill=True, **kw)
        for seed, T in ((13, 30), (14, 55)):      # the second prompt is longer than the ring
            ids = torch.randint(2, 96, (T,), generator=torch.Generator().manual_seed(seed)).to(DEV)
            want = torch.cat(list(plain.generate(ids, 24)))
            got = torch.cat(list(recorded.generate(ids, 24)))
            say(f"prompt of {T}: {want.numel()} tokens, recorded equal: {torch.equal(want, got)}")
            assert torch.equal(want, got)
            assert torch.equal(plain.history, recorded.history)
        # the reference's default cache dtype (fp16): the ring is streamed and appended to in place
        # all the same, and holds the same values (bf16 rows convert to fp16 without loss)
        kw.pop("dtype")
        default = Generator(model, **kw)
        assert default.cache.dtype == torch.float16 and default.use_ring_context
        assert torch.equal(torch.cat(list(default.generate(ids, 24))), want)
        assert torch.equal(default.cache.k.float(), plain.cache.k.float()) and torch.equal(default.cache.v.float(), plain.cache.v.float())


def test_generator_generate_batch():
    """Generator.generate_batch: greedy equals core.generate_greedy; sampling settings apply per row and a
    seed reproduces the draw; the repetition penalty of a batch equals the penalty row by row."""
    from daisy_amd import Generator
    from daisy_amd.generate import penalise_repeats
    with torch.no_grad():
        model = _Core().to(DEV)
        B, T = 3, 40
        ids = torch.randint(2, 96, (B, T), generator=torch.Generator().manual_seed(7)).to(DEV)
        gen = Generator(model, window=model.window_size, seed=3, device=torch.device(DEV), dtype=torch.bfloat16, temperature=0.0)
        out = gen.generate_batch(ids, 6)
        assert out.shape == (B, 6) and torch.equal(out, core.generate_greedy(model, ids, 6))
        for _ in range(2):   # recorded on the first call, replayed on the second
            assert torch.equal(gen.generate_batch(ids, 6, record_steps=True), out), "recorded steps change the tokens"
        gen.set_temperature(0.8)
        gen.top_k, gen.top_p = 20, 0.9
        gen.set_repetition_penalty(1.3)
        torch.manual_seed(11)
        a = gen.generate_batch(ids, 5)
        torch.manual_seed(11)
        b = gen.generate_batch(ids, 5)
        assert torch.equal(a, b) and int(a.min()) >= 0 and int(a.max()) < 96
        logits = torch.randn(B, 96, device=DEV)
        recent = torch.randint(0, 96, (B, 17), device=DEV)
        batch = penalise_repeats(logits, recent, gen.rep_p_t.float())
        for r in range(B):
            assert torch.allclose(batch[r], penalise_repeats(logits[r], recent[r], gen.rep_p_t.float()), rtol=1e-6, atol=1e-6)


def test_recorded_steps_survive_alternating_batch_sizes_on_a_hybrid_stack():
    """A recorded step carries raw addresses of the KDA layer's state.  One sequence with recorded steps,
    then a batch of four, then one sequence again: the states of the two batch sizes live in buffers of
    their own, every recording is checked against the current addresses before it is replayed, and the
    tokens equal those of steps launched kernel by kernel."""
    import copy
    from daisy_amd import Generator, KimiLinearSelfAttention
    with torch.no_grad():
        model = _Core(window=48, max_seq_len=512)
        torch.manual_seed(2)
        model.blocks[0].attn = KimiLinearSelfAttention(256, 2, 512, 128, receives_ve=True).bfloat16()
        model = model.to(DEV)
        twin = copy.deepcopy(model)
        kw = dict(window=48, seed=5, device=torch.device(DEV), dtype=torch.bfloat16, temperature=0.0)
        plain, recorded = Generator(model, **kw), Generator(twin, record_steps=True, direct_prefill=True, **kw)
        g = torch.Generator().manual_seed(21)
        one_a = torch.randint(2, 96, (33,), generator=g).to(DEV)
        four = torch.randint(2, 96, (4, 27), generator=g).to(DEV)
        one_b = torch.randint(2, 96, (40,), generator=g).to(DEV)
        for round_ in range(2):
            say(f"alternating batch sizes, round {round_}: one sequence")
            assert torch.equal(torch.cat(list(recorded.generate(one_a, 16))), torch.cat(list(plain.generate(one_a, 16))))
            state_1 = twin.blocks[0].attn._recurrent_state
            say(f"alternating batch sizes, round {round_}: batch of four")
            assert torch.equal(recorded.generate_batch(four, 12, record_steps=True), plain.generate_batch(four, 12))
            assert twin.blocks[0].attn._recurrent_state.shape[0] == 4
            say(f"alternating batch sizes, round {round_}: one sequence again")
            assert torch.equal(torch.cat(list(recorded.generate(one_b, 16))), torch.cat(list(plain.generate(one_b, 16))))
            # the one-sequence state went back into the buffer it had before the batch of four came by
            assert twin.blocks[0].attn._recurrent_state.data_ptr() == state_1.data_ptr()
        recorded._recorded_step.check()                      # no step ran past the rotary tables
        # a step recorded without a prefill would capture the creation of the layer's state: refused
        twin.reset_history()
        twin.blocks[0].attn._state_homes.clear()
        # (inference mode like the generators above: torch keeps per-capture generator state that must be
        # touched in the mode it was created in)
        with torch.inference_mode(), pytest.raises(RuntimeError, match="in place"):
            core.GraphedStep(twin, KVCache(4, 1, 2, 48, 128, DEV, torch.bfloat16))(one_a[:1])
