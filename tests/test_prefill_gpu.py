"""Kernel 1 parity: HIP prefill attention vs the fp32 oracle (through the C ABI)."""
import pytest
import torch

import oracle
from daisy_amd import ops
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu


def _inputs(B, T, H, D, seed, normalise=False):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(B, T, H, D, generator=g) for _ in range(3))
    if normalise:
        q, k, v = (oracle.rms_norm(t) for t in (q, k, v))
    return q.bfloat16(), k.bfloat16(), v.bfloat16()


def _oracle(q, k, v, window, cos=None, sin=None, doc_start=None, scale=0.12, rows=None):
    if cos is not None:
        q, k = oracle.apply_rope(q, cos, sin), oracle.apply_rope(k, cos, sin)
    q_, k_, v_ = (t.transpose(1, 2) for t in (q, k, v))
    if rows is None and q.shape[1] <= 2048:
        o = oracle.windowed_attention(q_, k_, v_, window, scale, doc_start)
    else:
        o = oracle.windowed_attention_blockwise(q_, k_, v_, window, scale, doc_start, rows=rows)
    return o.transpose(1, 2), k


CASES = [
    # B, T, H, D, window, rope, docs
    (1, 256, 4, 64, 128, True, False),      # plumbing config shape
    (2, 512, 2, 128, 200, True, False),
    (1, 300, 3, 128, 64, True, True),       # ragged T, documents
    (1, 129, 1, 128, None, False, False),   # full causal, one row past a block
    (2, 64, 2, 64, 1, False, False),        # window 1: every query sees only itself
    (1, 1, 1, 128, 16, True, False),        # single token
    (1, 1000, 2, 128, 1000, True, True),    # window == T
    (1, 96, 2, 8, 16, True, True),          # scalar kernel (small head dim)
    (1, 40, 1, 2, None, True, False),       # scalar kernel, head dim 2 (no truncation in the tables)
    # longer sequences: many tiles per query block, rotated tile order with a wrap
    (1, 1111, 2, 128, 300, True, True),     # ragged T, documents, window shorter than a block
    (2, 1024, 1, 64, 1000, True, False),    # head dim 64, window just under T
    (1, 1300, 2, 128, None, False, False),  # full causal
    (1, 2048, 1, 128, 64, False, True),     # window of one tile: most tiles of a block are skipped
]


@pytest.mark.parametrize("B,T,H,D,window,rope,docs", CASES)
def test_prefill_matches_oracle(B, T, H, D, window, rope, docs):
    say(f"prefill case B{B} T{T} H{H} D{D} W{window} rope={rope} docs={docs}")
    q, k, v = _inputs(B, T, H, D, seed=T + D)
    cos = sin = doc_start = None
    if rope:
        cos, sin = oracle.rope_tables(D, T + 5)
    if docs:
        ids = torch.randint(0, 7, (T,), generator=torch.Generator().manual_seed(1))
        doc_start = oracle.doc_start_from_ids(ids, 3)
    ref, k_ref = _oracle(q, k, v, window, None if cos is None else cos[:T], None if sin is None else sin[:T], doc_start)
    dev = "cuda:0"
    o, k_rot = ops.prefill_attention(
        q.to(dev), k.to(dev), v.to(dev), window=window,
        cos=None if cos is None else cos.to(dev), sin=None if sin is None else sin.to(dev),
        doc_start=None if doc_start is None else doc_start.to(dev))
    torch.cuda.synchronize()
    assert_close_bf16(o, ref, "o")
    if rope:
        bad = (k_rot.cpu() != k_ref)
        assert not bad.any(), (f"rotated keys must be bit-identical to the oracle's bf16 RoPE: {int(bad.sum())} of "
                               f"{bad.numel()} differ, max diff {(k_rot.cpu().float() - k_ref.float()).abs().max().item():.3e}")
    else:
        assert k_rot is None


def test_prefill_strided_views_of_merged_qkv():
    """q, k, v as chunks of one [B, T, 3H, D] projection output, as the module passes them."""
    B, T, H, D = 2, 384, 4, 128
    g = torch.Generator().manual_seed(7)
    qkv = torch.randn(B, T, 3 * H, D, generator=g).bfloat16()
    q, k, v = qkv.chunk(3, dim=-2)
    cos, sin = oracle.rope_tables(D, T)
    ref, _ = _oracle(q, k, v, 100, cos, sin)
    dq = qkv.to("cuda:0")
    q2, k2, v2 = dq.chunk(3, dim=-2)
    o, _ = ops.prefill_attention(q2, k2, v2, window=100, cos=cos.cuda(), sin=sin.cuda())
    assert_close_bf16(o, ref, "o")


@pytest.mark.parametrize("H,D,T", [(4, 128, 333), (3, 128, 200), (2, 64, 130)])
def test_prefill_outputs_with_caller_strides(H, D, T):
    """o and the rotated keys written into views with other strides ([B, H, T, D] storage, the ring's
    layout; rows of a wider buffer) equal the contiguous results bit for bit, and nothing outside the
    views is touched.  Odd H takes the one-head-per-thread pre-pass, even H the two-head one."""
    B, W = 2, 70
    q, k, v = (t.cuda() for t in _inputs(B, T, H, D, seed=21))
    cos, sin = (t.cuda() for t in oracle.rope_tables(D, T))
    o_ref, k_ref = ops.prefill_attention(q, k, v, window=W, cos=cos, sin=sin)
    # [B, H, T, D] storage seen as [B, T, H, D]
    o_bhtd = torch.full((B, H, T, D), 7.0, dtype=torch.bfloat16, device="cuda:0")
    k_bhtd = torch.full((B, H, T, D), 7.0, dtype=torch.bfloat16, device="cuda:0")
    ops.prefill_attention(q, k, v, window=W, cos=cos, sin=sin, out=o_bhtd.transpose(1, 2), k_out=k_bhtd.transpose(1, 2))
    assert torch.equal(o_bhtd.transpose(1, 2), o_ref) and torch.equal(k_bhtd.transpose(1, 2), k_ref)
    # rows of a wider buffer: [B, T, H, D + 16] with the last 16 channels of every row left alone
    o_wide = torch.full((B, T, H, D + 16), 7.0, dtype=torch.bfloat16, device="cuda:0")
    k_wide = torch.full((B, T, H, D + 16), 7.0, dtype=torch.bfloat16, device="cuda:0")
    ops.prefill_attention(q, k, v, window=W, cos=cos, sin=sin, out=o_wide[..., :D], k_out=k_wide[..., :D])
    assert torch.equal(o_wide[..., :D], o_ref) and torch.equal(k_wide[..., :D], k_ref)
    assert bool((o_wide[..., D:] == 7.0).all()) and bool((k_wide[..., D:] == 7.0).all())
    say(f"strided outputs H={H} D={D} T={T}: equal to the contiguous results")


def test_prefill_long_sequence_sampled_rows():
    """T = 16384 with a 2048 window: spot-check rows against the blockwise oracle."""
    B, T, H, D, W = 1, 16384, 2, 128, 2048
    q, k, v = _inputs(B, T, H, D, seed=3)
    rows = torch.cat([torch.arange(0, 64), torch.arange(2040, 2060), torch.arange(8000, 8032), torch.arange(T - 64, T)])
    ref, _ = _oracle(q, k, v, W, rows=rows)
    o, _ = ops.prefill_attention(q.cuda(), k.cuda(), v.cuda(), window=W)
    assert_close_bf16(o[:, rows.cuda()], ref, "o[rows]")


def test_prefill_is_deterministic_and_window_invariant():
    """A window >= T equals full causal attention bit for bit; repeated calls agree."""
    B, T, H, D = 1, 320, 2, 128
    q, k, v = (t.cuda() for t in _inputs(B, T, H, D, seed=11))
    a, _ = ops.prefill_attention(q, k, v, window=None)
    b, _ = ops.prefill_attention(q, k, v, window=T)
    c, _ = ops.prefill_attention(q, k, v, window=T + 1000)
    assert torch.equal(a, b) and torch.equal(a, c)


def test_prefill_rejects_bad_arguments():
    q = torch.zeros(1, 8, 1, 64, dtype=torch.bfloat16, device="cuda:0")
    with pytest.raises(RuntimeError, match="head_dim"):
        ops.prefill_attention(torch.zeros(1, 8, 1, 7 * 2 + 1, dtype=torch.bfloat16, device="cuda:0"),
                              torch.zeros(1, 8, 1, 15, dtype=torch.bfloat16, device="cuda:0"),
                              torch.zeros(1, 8, 1, 15, dtype=torch.bfloat16, device="cuda:0"), window=4)
    with pytest.raises(TypeError):
        ops.prefill_attention(q.float(), q.float(), q.float(), window=4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.prefill_attention(q.cpu(), q.cpu(), q.cpu(), window=4)
