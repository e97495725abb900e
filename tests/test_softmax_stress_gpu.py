"""Online-softmax stress for kernels 1 and 2: logits whose running row maximum moves a lot.

The ordinary parity cases use scale 0.12 on unit-variance inputs: scores a few log2 units wide, so the
rescale of the running sums almost never fires after a row's first tile.  Here scale = 1 and the keys are
built so that the score of a (query, key) pair grows (or falls) steadily with the key's position: the row
maximum rises tile after tile by a chosen amount -- below the kernels' lazy-rescale threshold (2^8), just
above it, and far above it (old contributions scaled by ~2^-40) -- or sits in the first / last key a query
sees.  Checked against the fp32 oracle at the usual bf16 tolerances.
"""
import pytest
import torch

import oracle
from daisy_amd import ops
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu

LOG2E = 1.4426950408889634


def _structured(B, T, H, D, rise_per_32_keys, seed, noise=0.3):
    """q, k, v [B, T, H, D] bf16 with  <q_i, k_j> ~= c * j  (+ noise of a few units), where c makes the score,
    in log2 units, move by `rise_per_32_keys` over 32 consecutive keys (negative: the score falls with j)."""
    g = torch.Generator().manual_seed(seed)
    u = torch.nn.functional.normalize(torch.randn(B, 1, H, D, generator=g), dim=-1)
    a = 4.0
    j = torch.arange(T, dtype=torch.float32).view(1, T, 1, 1)
    slope = rise_per_32_keys / 32.0 / LOG2E / a            # natural-log units per key, divided by |q . u|
    q = a * u + noise * torch.randn(B, T, H, D, generator=g)
    k = slope * j * u + noise * torch.randn(B, T, H, D, generator=g)
    v = torch.randn(B, T, H, D, generator=g)
    return q.bfloat16(), k.bfloat16(), v.bfloat16()


def _random_large(B, T, H, D, seed):
    """q, k ~ 3 N(0,1) (scores hundreds of log2 units apart), v ~ N(0,1) (outputs of a size at which the rounding of
    the bf16 result itself stays well inside the tolerance)."""
    g = torch.Generator().manual_seed(seed)
    q, k = ((3.0 * torch.randn(B, T, H, D, generator=g)).bfloat16() for _ in range(2))
    return q, k, torch.randn(B, T, H, D, generator=g).bfloat16()


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("window", [None, 200, 1])
@pytest.mark.parametrize("rise", [5.0, 12.0, 40.0, -12.0, -40.0, "random"])
def test_prefill_large_logits(D, window, rise):
    """T = 700: 5.5 query blocks, 22 key tiles; with window 200 the tile order is rotated (every block starts in
    the middle of its range and wraps), so a rising score puts the row maximum in a tile that is visited in the
    middle of the walk and a falling one in the tile visited right after the wrap."""
    if window == 1 and rise not in (5.0, "random"):
        pytest.skip("one key per row: the structure does not matter")
    B, T, H = 1, 700, 2
    say(f"prefill large logits D{D} window {window} rise {rise}")
    q, k, v = _random_large(B, T, H, D, seed=D) if rise == "random" else _structured(B, T, H, D, rise, seed=D + 1)
    ref = oracle.windowed_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), window, 1.0).transpose(1, 2)
    s = torch.einsum("bihd,bjhd->bhij", q.float(), k.float()) * LOG2E
    say(f"  score range in log2 units: {s.min().item():.0f} .. {s.max().item():.0f}")
    o, _ = ops.prefill_attention(q.cuda(), k.cuda(), v.cuda(), window=window, scale=1.0)
    assert_close_bf16(o, ref, "o")


@pytest.mark.parametrize("D", [64, 128])
def test_prefill_large_logits_with_rotation_and_documents(D):
    """The same with RoPE in the call and document bounds (masked tiles take the same softmax path)."""
    B, T, H, W = 2, 515, 2, 300
    q, k, v = _random_large(B, T, H, D, seed=7 * D)
    cos, sin = oracle.rope_tables(D, T)
    doc_start = torch.zeros(T, dtype=torch.int32)
    doc_start[130:] = 130
    doc_start[401:] = 401
    qr, kr = oracle.apply_rope(q, cos, sin), oracle.apply_rope(k, cos, sin)
    ref = oracle.windowed_attention(qr.transpose(1, 2), kr.transpose(1, 2), v.transpose(1, 2), W, 1.0, doc_start).transpose(1, 2)
    o, _ = ops.prefill_attention(q.cuda(), k.cuda(), v.cuda(), window=W, scale=1.0, cos=cos.cuda(), sin=sin.cuda(),
                                 doc_start=doc_start.cuda())
    assert_close_bf16(o, ref, "o")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("nsplit", [0, 1, 5])
@pytest.mark.parametrize("rise", [5.0, 12.0, 40.0, -40.0, "random"])
def test_decode_large_logits(D, nsplit, rise):
    """One query over a ring of 1000 rows whose scores rise / fall with the slot index (the kernel streams the ring
    in physical order, every lane group and every split keeps its own running maximum, and the merges across lane
    groups, wavefronts and splits see partial maxima that are far apart)."""
    B, H, W = 2, 3, 1000
    say(f"decode large logits D{D} nsplit {nsplit} rise {rise}")
    if rise == "random":
        _, kc, vc = _random_large(B, W, H, D, seed=D + 3)
        q = (3.0 * torch.randn(B, H, D, generator=torch.Generator().manual_seed(5))).bfloat16()
    else:
        q_all, kc, vc = _structured(B, W, H, D, rise, seed=D + 4)
        q = q_all[:, 0]
    kc, vc = kc.transpose(1, 2).contiguous(), vc.transpose(1, 2).contiguous()     # [B, H, W, D]
    g = torch.Generator().manual_seed(11)
    kn, vn = ((torch.randn(B, H, D, generator=g)).bfloat16() for _ in range(2))
    slot = 617
    k_exp, v_exp = kc.clone(), vc.clone()
    k_exp[:, :, slot], v_exp[:, :, slot] = kn, vn
    ref = oracle.sdpa(q[:, :, None], k_exp, v_exp, None, 1.0)[:, :, 0]
    o = ops.decode_attention(q.cuda(), kn.cuda(), vn.cuda(), kc.cuda(), vc.cuda(), n_rows=W, new_idx=slot,
                             write_back=True, scale=1.0, nsplit=nsplit)
    assert_close_bf16(o, ref, "o")
