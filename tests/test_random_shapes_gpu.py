"""Seeded sweep over ragged shapes: each kernel against the oracle on sizes the tests with named
cases do not list (lengths around the 16/64/128 tile edges, windows shorter and longer than the
sequence, documents, strided q/k/v views of one projection output, rings of odd sizes at
positions before and after the wrap, host- and device-side positions, KDA sequences that end inside
a chunk, steep gates, bf16 gates, carried states)."""
import random

import pytest
import torch

import oracle
from oracle import kda as okda
from daisy_amd import chunk_kda, fused_recurrent_kda, ops
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu
SCALE = 0.12


@pytest.mark.parametrize("seed", [11, 12])
def test_prefill_random_shapes(seed):
    rng = random.Random(seed)
    for it in range(60):
        B, H, D = rng.choice([1, 1, 2, 3]), rng.choice([1, 2, 3, 5]), rng.choice([128, 128, 64])
        T = rng.choice([1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 191, 255, 256, 257, 300, 383, 385, 511, 513, 640])
        window = rng.choice([None, 1, 2, 16, 17, 64, 100, 127, 128, 129, 200, 256, 300, 512, 1000])
        rope, docs, strided = rng.random() < 0.6, rng.random() < 0.5, rng.random() < 0.4
        if rope:
            rng.random()   # one draw more for rotated cases (keeps the case sequence of this seed unchanged)
        say(f"prefill sweep seed {seed} case {it}: B{B} H{H} D{D} T{T} window {window} rope {rope} docs {docs} "
            f"strided {strided}")
        g = torch.Generator().manual_seed(seed * 100003 + it)
        if strided:   # three views of one [B, T, 3H, D] tensor, the layout of the QKV projection output
            qkv = torch.randn(B, T, 3 * H, D, generator=g).bfloat16()
            q, k, v = qkv.chunk(3, dim=2)
            qd, kd, vd = qkv.cuda().chunk(3, dim=2)
        else:
            q, k, v = (torch.randn(B, T, H, D, generator=g).bfloat16() for _ in range(3))
            qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
        doc_start = None
        if docs:
            doc_start = torch.zeros(T, dtype=torch.int32)
            for c in sorted({rng.randrange(0, T) for _ in range(rng.choice([1, 2, 5]))}):
                doc_start[c:] = c
        cos = sin = None
        qr, kr = q, k
        if rope:
            cos, sin = oracle.rope_tables(D, T + rng.choice([0, 5]))
            qr, kr = oracle.apply_rope(q, cos[:T], sin[:T]), oracle.apply_rope(k, cos[:T], sin[:T])
        ref = oracle.windowed_attention(qr.transpose(1, 2), kr.transpose(1, 2), v.transpose(1, 2), window, SCALE,
                                        doc_start).transpose(1, 2)
        o, k_rot = ops.prefill_attention(qd, kd, vd, window=window, scale=SCALE,
                                         cos=None if cos is None else cos.cuda(), sin=None if sin is None else sin.cuda(),
                                         doc_start=None if doc_start is None else doc_start.cuda())
        assert_close_bf16(o, ref, f"o (case {it})")
        if rope:
            assert_close_bf16(k_rot, kr, f"rotated keys (case {it})")


@pytest.mark.parametrize("seed", [21, 22])
def test_decode_random_rings(seed):
    rng = random.Random(seed)
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    for it in range(80):
        B, H, D = rng.choice([1, 2, 5]), rng.choice([1, 3, 4]), rng.choice([128, 128, 64])
        W = rng.choice([1, 2, 7, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 255, 256, 257, 511, 512, 513, 1024, 1500, 2048, 4096, 5000])
        t = rng.choice([0, 1, W - 1, W, W + 1, 2 * W, rng.randrange(0, 3 * W + 1), rng.randrange(0, W + 1)])
        nsplit, on_device = rng.choice([0, 0, 1, 2, 3, 7, 16, 40, 64]), rng.random() < 0.5
        say(f"decode sweep case {it}: B{B} H{H} D{D} W{W} t{t} nsplit{nsplit} position on device {on_device}")
        g = torch.Generator().manual_seed(seed * 7919 + it)
        kc, vc = (torch.randn(B, H, W, D, generator=g).bfloat16() for _ in range(2))
        q, kn, vn = (torch.randn(B, H, D, generator=g).bfloat16() for _ in range(3))
        n_rows, slot = min(t + 1, W), t % W
        k_exp, v_exp = kc.clone(), vc.clone()
        k_exp[:, :, slot], v_exp[:, :, slot] = kn, vn
        ref = oracle.sdpa(q[:, :, None, :], k_exp[:, :, :n_rows], v_exp[:, :, :n_rows], None, SCALE)[:, :, 0, :]
        dk, dv = kc.cuda(), vc.cuda()
        if on_device:
            pos.fill_(t)
            o = ops.decode_attention_at(q.cuda(), kn.cuda(), vn.cuda(), dk, dv, pos, nsplit=nsplit)
        else:
            o = ops.decode_attention(q.cuda(), kn.cuda(), vn.cuda(), dk, dv, n_rows=n_rows, new_idx=slot,
                                     write_back=True, nsplit=nsplit)
        assert_close_bf16(o, ref, f"o (case {it})")
        assert torch.equal(dk.cpu(), k_exp) and torch.equal(dv.cpu(), v_exp), f"ring contents (case {it})"


@pytest.mark.parametrize("seed", [31])
def test_kda_random_sequences(seed):
    rng = random.Random(seed)
    for it in range(24):
        B, H = rng.choice([1, 2]), rng.choice([1, 2, 3])
        T = rng.choice([1, 2, 15, 16, 17, 63, 64, 65, 100, 127, 128, 129, 200, 257])
        steep, g_bf16, carried, token_by_token = (rng.random() < p for p in (0.4, 0.4, 0.5, 0.25))
        say(f"kda sweep case {it}: B{B} H{H} T{T} steep {steep} bf16 gate {g_bf16} carried state {carried} "
            f"token by token {token_by_token}")
        gen = torch.Generator().manual_seed(seed * 104729 + it)
        q, k, v = (torch.randn(B, T, H, 128, generator=gen).bfloat16() for _ in range(3))
        gate = torch.nn.functional.logsigmoid(torch.randn(B, T, H, 128, generator=gen))
        if steep:   # the decay rates of a KDA layer at initialisation: up to 16 times faster per head
            gate = gate * torch.empty(1, 1, H, 1).uniform_(1, 16, generator=gen)
        if g_bf16:
            gate = gate.bfloat16()
        beta = torch.sigmoid(torch.randn(B, T, H, generator=gen))
        s0 = torch.randn(B, H, 128, 128, generator=gen) * 0.5 if carried else None
        o_ref, s_ref = okda.kda_recurrent(q, k, v, gate.float(), beta, initial_state=s0)
        fn = fused_recurrent_kda if token_by_token else chunk_kda
        o, s = fn(q.cuda(), k.cuda(), v.cuda(), gate.cuda(), beta.cuda(), initial_state=None if s0 is None else s0.cuda(),
                  output_final_state=True, use_qk_l2norm_in_kernel=True)
        assert_close_bf16(o, o_ref, f"o (case {it})")
        rel = ((s.cpu() - s_ref).norm() / s_ref.norm().clamp_min(1e-20)).item()
        assert torch.isfinite(s).all() and rel <= 1e-3, f"final state (case {it}): relative error {rel:.3e}"
