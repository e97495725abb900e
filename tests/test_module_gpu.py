"""Drop-in module parity on the GPU: CausalSelfAttention.forward/prefill/step,
KVCache ring decode and the Generator, against the CPU oracle."""
import os

import pytest
import torch
import torch.nn as nn

os.environ["DISABLE_O_ZERO_INIT"] = "1"

import oracle
from daisy_amd import CausalSelfAttention, Generator, KVCache, WindowMask, build_window_mask
from daisy_amd.functional import norm
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _make(dim, H, D, receives_ve=False, seed=0, max_seq_len=4096):
    torch.manual_seed(seed)
    attn = CausalSelfAttention(dim=dim, num_heads=H, head_dim=D, receives_ve=receives_ve, max_seq_len=max_seq_len)
    with torch.no_grad():
        attn.qkvo_w.copy_((torch.randn(4, dim, dim) * 0.02).bfloat16())
    return attn.eval()


def test_library_rms_norm_on_gpu_matches_oracle():
    """The projection outputs are normalised by the library routine on the GPU; pin its epsilon there too."""
    x = (torch.randn(4, 7, 3, 128, generator=torch.Generator().manual_seed(0)) * 1e-3).bfloat16()
    assert torch.equal(norm(x.to(DEV)).cpu(), oracle.rms_norm(x))
    x = torch.randn(4, 7, 3, 64, generator=torch.Generator().manual_seed(1)).bfloat16()
    assert (norm(x.to(DEV)).cpu().float() - oracle.rms_norm(x).float()).abs().max().item() <= 2 ** -7


def test_config1_plumbing_layer():
    """BASELINE config 1: B1 T256 d256 H4 D64 W128, fp32 x, weights N(0, 0.02), seed 0:
    the oracle's fp32 CPU path vs the HIP path (bf16 compute)."""
    torch.manual_seed(0)
    dim, H, D, T, W = 256, 4, 64, 256, 128
    w = torch.randn(4, dim, dim) * 0.02
    x = torch.randn(1, T, dim)
    for base, trunc in ((10000.0, False), (1024.0, True)):
        cos, sin = oracle.rope_tables(D, T, base=base, half_truncate=trunc)
        # The reference's CPU path: its parameters are bf16 (models/daisy/attention.py:82) and x is cast to them.
        y_ref, k_ref, v_ref = oracle.attn_prefill(x, w.bfloat16(), H, D, cos, sin, W)
        y_f32, _, _ = oracle.attn_prefill(x, w, H, D, cos, sin, W)           # the same layer with nothing rounded
        attn = _make(dim, H, D)
        with torch.no_grad():
            attn.qkvo_w.copy_(w.bfloat16())
            attn.rotary.cos[:T].copy_(cos)
            attn.rotary.sin[:T].copy_(sin)
        attn = attn.to(DEV)
        y, k, v = attn.prefill(x.to(DEV), None, attn_mask=WindowMask(W))
        assert y.shape == (1, T, dim) and k.shape == (1, H, T, D) and v.shape == (1, H, T, D)
        assert y.dtype == torch.bfloat16
        assert_close_bf16(y, y_ref, f"y (base {base})")
        assert_close_bf16(y, y_f32, f"y vs the unrounded layer (base {base})")
        assert_close_bf16(k, k_ref, "k")
        assert_close_bf16(v, v_ref, "v")


@pytest.mark.parametrize("fused_prep", [True, False])
@pytest.mark.parametrize("receives_ve", [False, True])
def test_prefill_matches_oracle_with_documents_and_ve(receives_ve, fused_prep):
    dim, H, D, T, W = 512, 4, 128, 333, 100
    attn = _make(dim, H, D, receives_ve=receives_ve, seed=1).to(DEV)
    attn.fused_prep = fused_prep    # one-pass norm + RoPE + mix kernel, or the library ops + RoPE inside attention
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, T, dim, generator=g).bfloat16()
    ve = torch.randn(2, T, dim, generator=g).bfloat16() if receives_ve else None
    ids = torch.randint(0, 6, (1, T), generator=g)
    w = attn.qkvo_w.detach().cpu()
    cos, sin = attn.rotary.cos.cpu(), attn.rotary.sin.cpu()
    y_ref, k_ref, v_ref = oracle.attn_prefill(x, w, H, D, cos, sin, W, doc_start=oracle.doc_start_from_ids(ids, 3),
                                              ve=ve, g_ve=0.0 if receives_ve else None)
    mask = build_window_mask(ids.to(DEV), W, 3)
    y, k, v = attn.prefill(x.to(DEV), None if ve is None else ve.to(DEV), attn_mask=mask)
    assert_close_bf16(y, y_ref, "y")
    assert_close_bf16(k, k_ref, "k")
    assert_close_bf16(v, v_ref, "v")
    # the reference's dense additive mask is accepted too and means the same thing
    dense = oracle.build_attn_mask(ids, W, 3).to(DEV)
    # (per-row lower bounds instead of a window: the kernel visits the key tiles in another order,
    # so the two results agree to rounding, not bit for bit)
    y2 = attn(x.to(DEV), None if ve is None else ve.to(DEV), attn_mask=dense)
    assert_close_bf16(y2, y, "dense mask vs descriptor", max_abs=8e-3, mean_abs=2e-4)
    assert_close_bf16(y2, y_ref, "y (dense mask)")


@pytest.mark.parametrize("T,W,fused_prep", [(128, 128, True), (131, 128, True), (70, 16, True), (70, 16, False)])
def test_forward_equals_steps(T, W, fused_prep):
    """Reference tests/test_causal_self_attention_equivalence.py: full forward == T streaming steps (bf16, 2e-2)."""
    dim, H, D = 128, 2, 64
    attn = _make(dim, H, D, receives_ve=True, seed=3).to(DEV)
    attn.fused_prep = fused_prep
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, T, dim, generator=g).bfloat16().to(DEV)
    ve = torch.randn(1, T, H, D, generator=g).bfloat16().to(DEV)
    y_full = attn(x, ve, attn_mask=WindowMask(W))
    K = torch.empty(1, 0, H, D, device=DEV, dtype=torch.bfloat16)
    V = torch.empty(1, 0, H, D, device=DEV, dtype=torch.bfloat16)
    ys = []
    for pos in range(T):
        y, k_new, v_new = attn.step(x[:, pos:pos + 1], k_ctx=K, v_ctx=V, pos=pos, ve=ve[:, pos:pos + 1], window=W)
        assert y.shape == (1, 1, dim) and k_new.shape == (1, 1, H, D)
        K, V = torch.cat([K, k_new], 1), torch.cat([V, v_new], 1)
        ys.append(y)
    y_step = torch.cat(ys, 1)
    assert torch.allclose(y_full.float(), y_step.float(), atol=2e-2, rtol=2e-2), \
        f"max err {(y_full.float() - y_step.float()).abs().max().item()}"


def test_step_ring_context_equals_chronological_context():
    """The in-place ring path and the reference's tensor path give the same step, and the ring gets the new row."""
    dim, H, D, W, B = 256, 2, 128, 32, 3
    attn = _make(dim, H, D, seed=5).to(DEV)
    g = torch.Generator().manual_seed(6)
    cache_a = KVCache(L=1, B=B, H=H, W=W, D=D, device=DEV, dtype=torch.bfloat16)
    cache_b = KVCache(L=1, B=B, H=H, W=W, D=D, device=DEV, dtype=torch.bfloat16)
    for t in range(W + 9):     # wraps the ring
        x = torch.randn(B, 1, dim, generator=g).bfloat16().to(DEV)
        ring = cache_a.ring(0)
        ya, ka, va = attn.step(x, ring, ring, t, None, window=W)
        assert cache_a._staged[0] is True          # the kernel appended the row itself
        cache_a.advance()
        kc, vc = cache_b.view(0)
        yb, kb, vb = attn.step(x, kc, vc, t, None, window=W)
        cache_b.write(0, kb, vb)
        cache_b.advance()
        assert_close_bf16(ya, yb.float(), f"y at t={t}", max_abs=1e-2, mean_abs=1e-3)
        assert torch.equal(ka, kb) and torch.equal(va, vb)
    assert torch.equal(cache_a.k, cache_b.k) and torch.equal(cache_a.v, cache_b.v)


class TinyModel(nn.Module):
    """Two attention layers + embeddings, with the model-level prefill/step contract the Generator needs."""

    def __init__(self, vocab=64, dim=128, H=2, D=64, window=16):
        super().__init__()
        self.eos_token_id = vocab - 1
        self.window = window
        self.embed = nn.Embedding(vocab, dim)
        self.blocks = nn.ModuleList([nn.Module() for _ in range(2)])
        for i, b in enumerate(self.blocks):
            b.attn = _make(dim, H, D, seed=10 + i, max_seq_len=512)
        self.head = nn.Linear(dim, vocab, bias=False)

    def reset_history(self):
        for b in self.blocks:
            b.attn.reset_history()

    def prefill(self, ids):
        x = norm(self.embed(ids)).bfloat16()
        mask = build_window_mask(ids, self.window, self.eos_token_id)
        ks, vs = [], []
        for b in self.blocks:
            y, k, v = b.attn.prefill(x, None, attn_mask=mask)
            x = x + y
            ks.append(k); vs.append(v)
        logits = self.head(norm(x)[:, -1].float())
        return logits, torch.stack([torch.stack(ks), torch.stack(vs)])

    def step(self, token, k_ctxs, v_ctxs, pos):
        x = norm(self.embed(token.view(1, 1))).bfloat16()
        ks, vs = [], []
        for i, b in enumerate(self.blocks):
            y, k, v = b.attn.step(x, k_ctxs[i], v_ctxs[i], pos, None, window=self.window)
            x = x + y
            ks.append(k); vs.append(v)
        return self.head(norm(x).float()).view(1, -1), ks, vs


def test_generator_ring_path_matches_full_prefill():
    """Greedy generation with the in-place ring path: every step's logits equal a fresh prefill of the whole
    sequence (same window semantics), so prefill -> cache -> step is consistent end to end."""
    torch.manual_seed(0)
    model = TinyModel().to(DEV).eval()
    gen = Generator(model, window=model.window, seed=1, device=torch.device(DEV), dtype=torch.bfloat16, temperature=0.0)
    assert gen.use_ring_context
    prompt = torch.randint(0, 60, (23,), generator=torch.Generator().manual_seed(3)).to(DEV)
    with torch.inference_mode():
        gen.reset_history()
        logits = gen._prefill(prompt)
        seq = prompt
        for _ in range(12):
            tok = torch.argmax(logits[-1])
            logits = gen._step(tok)
            seq = torch.cat([seq, tok.view(1)])
            want, _ = model.prefill(seq[None])
            assert torch.allclose(logits.float(), want.float(), atol=3e-2, rtol=3e-2), \
                f"step logits differ from prefill logits by {(logits.float() - want.float()).abs().max().item()}"
        assert gen.cache.t == seq.numel()
        out = [int(t) for t in gen.generate(prompt, max_new_tokens=5)]
        assert len(out) == 5


def test_forward_with_training_block_masks():
    """forward(block_mask=...) with the descriptors of build_block_window_masks equals dense attention under the
    reference's block-mask visibility (models/daisy/daisy_core.py:182-229), for the long and the short window."""
    from daisy_amd import build_block_window_masks
    dim, H, D, T, w_blocks, L = 256, 2, 128, 640, 3, 4
    attn = _make(dim, H, D, seed=5).to(DEV)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(1, T, dim, generator=g).bfloat16()
    ids = torch.randint(2, 40, (T,), generator=g)
    ids[[70, 300, 301, 511]] = 1
    masks = build_block_window_masks(ids.to(DEV), w_blocks, L, eos_token_id=1)
    widths = oracle.block_mask_cycle(L, w_blocks)
    w = attn.qkvo_w.detach().cpu()
    cos, sin = attn.rotary.cos.cpu(), attn.rotary.sin.cpu()
    q, k, v = oracle.calc_qkv(x, w, H, D, cos, sin)
    for layer in (0, 1):                       # long, short
        vis = oracle.block_mask_dense(ids, widths[layer], eos_token_id=1)
        add = torch.zeros(T, T).masked_fill(~vis, float("-inf"))
        o = oracle.sdpa(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), add, 0.12).transpose(1, 2)
        y_ref = torch.nn.functional.linear(o.reshape(1, T, dim).to(w.dtype), w[3])
        y = attn(x.to(DEV), None, block_mask=masks[layer])
        assert_close_bf16(y, y_ref, f"y (window of {widths[layer]} blocks)")


@pytest.mark.parametrize("dim,H,D,T,W", [(2, 1, 2, 131, 128), (16, 2, 8, 12, 12), (16, 2, 8, 8, 16), (16, 2, 8, 20, 2)])
def test_forward_equals_steps_at_the_reference_tests_shapes(dim, H, D, T, W):
    """The shapes of the reference's own unit tests (tests/test_causal_self_attention_equivalence.py:15-52: H=1, D=2;
    tests/test_attention.py:80-146: dim 16, H=2, D=8, window 2 included): head dims the fast kernels do not take."""
    attn = _make(dim, H, D, seed=7).to(DEV)
    with torch.no_grad():
        # projections of order 1; the output projection scaled so that y is of the order of the benchmark
        # configurations' outputs, for which the absolute tolerances are stated
        wt = torch.randn(4, dim, dim, generator=torch.Generator().manual_seed(8)) * 0.5
        wt[3] *= 0.25
        attn.qkvo_w.copy_(wt.bfloat16())
    x = torch.randn(1, T, dim, generator=torch.Generator().manual_seed(9)).bfloat16().to(DEV)
    y_full = attn(x, None, attn_mask=WindowMask(W))
    w = attn.qkvo_w.detach().cpu()
    y_ref, _, _ = oracle.attn_prefill(x.cpu(), w, H, D, attn.rotary.cos.cpu()[:T], attn.rotary.sin.cpu()[:T], W)
    assert_close_bf16(y_full, y_ref, "forward vs oracle")
    K = torch.empty(1, 0, H, D, device=DEV, dtype=torch.bfloat16)
    V = torch.empty(1, 0, H, D, device=DEV, dtype=torch.bfloat16)
    ys = []
    for pos in range(T):
        y, k_new, v_new = attn.step(x[:, pos:pos + 1], k_ctx=K, v_ctx=V, pos=pos, ve=None, window=W)
        K, V = torch.cat([K, k_new], 1), torch.cat([V, v_new], 1)
        ys.append(y)
    assert torch.allclose(y_full.float(), torch.cat(ys, 1).float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dim,H,D,T,W", [(16, 2, 8, 12, 12), (16, 2, 8, 8, 16), (16, 2, 8, 20, 2), (2, 1, 2, 40, 7),
                                         (128, 2, 64, 70, 16), (256, 2, 128, 33, None)])
@pytest.mark.parametrize("receives_ve", [False, True])
def test_fp32_parameters_run_in_fp32(dim, H, D, T, W, receives_ve):
    """The reference's own unit tests swap the parameters to fp32 and compare at 1e-4
    (tests/test_attention.py:9,80-146).  A module with fp32 parameters runs fp32 kernels here: forward,
    returned keys and values and the streaming steps all match the fp32 oracle at that tolerance."""
    attn = _make(dim, H, D, receives_ve=receives_ve, seed=21).float()
    with torch.no_grad():
        attn.qkvo_w.copy_(torch.randn(4, dim, dim, generator=torch.Generator().manual_seed(22)) * (0.5 if dim <= 16 else 0.05))
        if receives_ve:
            attn.g_ve.fill_(0.3228)
    attn = attn.to(DEV)
    assert attn.qkvo_w.dtype == torch.float32
    g = torch.Generator().manual_seed(23)
    x = torch.randn(2, T, dim, generator=g)
    ve = torch.randn(2, T, dim, generator=g) if receives_ve else None
    w = attn.qkvo_w.detach().cpu()
    cos, sin = attn.rotary.cos.cpu(), attn.rotary.sin.cpu()
    gv = 0.3228 if receives_ve else None
    y_ref, k_ref, v_ref = oracle.attn_prefill(x, w, H, D, cos, sin, W, ve=ve, g_ve=gv)
    dev = lambda t: None if t is None else t.to(DEV)
    y, k, v = attn.prefill(dev(x), dev(ve), attn_mask=WindowMask(W), debug=True)
    assert y.dtype == k.dtype == v.dtype == torch.float32
    for got, ref, what in ((y, y_ref, "y"), (k, k_ref, "k"), (v, v_ref, "v")):
        assert torch.allclose(got.cpu(), ref, rtol=1e-4, atol=1e-4), f"{what}: {(got.cpu() - ref).abs().max().item():.2e}"
    assert attn.last_q is not None and torch.allclose(attn.last_k.transpose(1, 2).cpu(), k_ref, atol=1e-4)
    K = torch.empty(2, 0, H, D, device=DEV)
    V = torch.empty(2, 0, H, D, device=DEV)
    ys = []
    for pos in range(T):
        ys_, k_new, v_new = attn.step(dev(x[:, pos:pos + 1]), K, V, pos, None if ve is None else dev(ve[:, pos:pos + 1]), window=W)
        assert ys_.dtype == torch.float32 and k_new.shape == (2, 1, H, D)
        K, V = torch.cat([K, k_new], 1), torch.cat([V, v_new], 1)
        ys.append(ys_)
    assert torch.allclose(torch.cat(ys, 1).cpu(), y_ref, rtol=1e-4, atol=1e-4)
    assert torch.allclose(K.transpose(1, 2).cpu(), k_ref, atol=1e-4) and torch.allclose(V.transpose(1, 2).cpu(), v_ref, atol=1e-4)


def test_forward_takes_the_flex_block_mask_of_the_training_forward():
    """forward(block_mask=BlockMask): the object the reference's DaisyCore.forward builds and passes
    (models/daisy/daisy_core.py:209-221,251-262) is converted to per-row bounds once and gives the
    output of the explicit descriptors."""
    from daisy_amd import build_block_window_masks
    from helpers import flex_block_mask
    dim, H, D, T, w_blocks = 256, 2, 128, 640, 3
    attn = _make(dim, H, D, seed=5).to(DEV)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(1, T, dim, generator=g).bfloat16().to(DEV)
    ids = torch.randint(2, 40, (T,), generator=g)
    ids[[70, 300, 301, 511]] = 1
    for w_ in (w_blocks, w_blocks // 2):
        bm = flex_block_mask(ids, w_, eos=1)
        y_bm = attn(x, None, block_mask=bm)
        y_desc = attn(x, None, block_mask=build_block_window_masks(ids.to(DEV), w_, 1, eos_token_id=1)[0])
        assert torch.equal(y_bm, y_desc)
        from daisy_amd.attention import _converted_masks
        assert _converted_masks.get(bm, lambda m: None) is not None       # the conversion is remembered per object


def test_debug_taps_keep_rotated_q_and_k():
    """prefill(debug=True) stores last_q and last_k as the reference does (attention.py:176-178)."""
    dim, H, D, T = 256, 2, 128, 50
    attn = _make(dim, H, D, seed=9).to(DEV)
    x = torch.randn(1, T, dim, generator=torch.Generator().manual_seed(1)).bfloat16()
    attn.prefill(x.to(DEV), None, attn_mask=WindowMask(16))
    assert attn.last_q is None and attn.last_k is None
    attn.prefill(x.to(DEV), None, attn_mask=WindowMask(16), debug=True)
    q_ref, k_ref, _ = oracle.calc_qkv(x, attn.qkvo_w.detach().cpu(), H, D, attn.rotary.cos.cpu(), attn.rotary.sin.cpu())
    assert_close_bf16(attn.last_q, q_ref, "last_q")
    assert_close_bf16(attn.last_k, k_ref, "last_k")
    attn.reset_history()
    assert attn.last_q is None and attn.last_k is None


def test_a_device_position_past_the_rotary_tables_is_reported():
    """With the position in device memory the host cannot refuse a step past the tables (the reference
    asserts it on the host, attention.py:66): the kernel reports it in a status word and its outputs are NaN."""
    from daisy_amd import ops
    from daisy_amd.functional import NORM_EPS_BF16
    B, H, D, W, rows = 2, 2, 128, 64, 40
    g = torch.Generator().manual_seed(3)
    raw = torch.randn(B, 3 * H, D, generator=g).bfloat16().to(DEV)
    kc, vc = (torch.randn(B, H, W, D, generator=g).bfloat16().to(DEV) for _ in range(2))
    cos, sin = (t.to(DEV) for t in oracle.rope_tables(D, rows))
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    pos = torch.full((1,), rows - 1, dtype=torch.int32, device=DEV)
    o = ops.attn_step(raw[:, :H], raw[:, H:2 * H], raw[:, 2 * H:], kc, vc, pos, cos=cos, sin=sin, eps=NORM_EPS_BF16, status=status)
    assert int(status.item()) == 0 and bool(torch.isfinite(o.float()).all())
    ops.raise_for_status(status)
    pos.fill_(rows)                                   # one past the last table row
    o = ops.attn_step(raw[:, :H], raw[:, H:2 * H], raw[:, 2 * H:], kc, vc, pos, cos=cos, sin=sin, eps=NORM_EPS_BF16, status=status)
    assert int(status.item()) == 1 and bool(torch.isnan(o.float()).all())
    with pytest.raises(RuntimeError, match="past the rotary tables"):
        ops.raise_for_status(status)
    status.zero_()
    q4 = raw.view(B, 1, 3 * H, D)
    qo, ko, vo = ops.qkv_prep(q4[:, :, :H], q4[:, :, H:2 * H], q4[:, :, 2 * H:], eps=NORM_EPS_BF16, cos=cos, sin=sin, pos0=pos, status=status)
    assert int(status.item()) == 1 and bool(torch.isnan(qo.float()).any()) and bool(torch.isfinite(vo.float()).all())
