"""Kernel 3 parity: chunked KDA (HIP) vs the naive fp32 recurrence (through the C ABI).

Tolerances: outputs max-abs <= 2e-2 and mean-abs <= 2e-3 (bf16 I/O), final state
relative Frobenius error <= 1e-3.
"""
import pytest
import torch
import torch.nn.functional as F

import oracle
from daisy_amd import chunk_kda, fused_kda_gate, fused_recurrent_kda, ops
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu

STATE_REL = 1e-3


def _inputs(B, T, H, seed, g_scale=1.0, D=128):
    g = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, T, H, D, generator=g), dim=-1).bfloat16()
    k = F.normalize(torch.randn(B, T, H, D, generator=g), dim=-1).bfloat16()
    v = torch.randn(B, T, H, D, generator=g).bfloat16()
    gl = F.logsigmoid(torch.randn(B, T, H, D, generator=g)) * g_scale
    beta = torch.sigmoid(torch.randn(B, T, H, generator=g))
    return q, k, v, gl, beta


def _check(o, S, o_ref, S_ref, what):
    assert_close_bf16(o, o_ref, f"{what}: o")
    rel = ((S.float().cpu() - S_ref).norm() / S_ref.norm()).item()
    say(f"{what}: state rel err {rel:.3e}")
    assert rel <= STATE_REL, f"{what}: state relative error {rel:.3e} > {STATE_REL}"


@pytest.mark.parametrize("B,T,H,g_scale", [
    (1, 64, 1, 1.0),      # exactly one chunk
    (1, 128, 2, 1.0),     # two chunks: state hand-over
    (2, 200, 2, 1.0),     # ragged last chunk
    (1, 17, 1, 1.0),      # shorter than a chunk
    (1, 512, 2, 0.05),    # slow decay: long memory, the S0 terms matter
    (1, 256, 2, 8.0),     # very fast decay (|g| up to ~50 per step): nothing may overflow; diagonal blocks decay
                          # beyond e^-80 over 16 rows and take the four-reference path on the matrix cores
    (1, 192, 2, 15.0),    # some groups of four rows decay beyond e^-80 by themselves, others do not
    (1, 256, 2, 30.0),    # most groups of four rows do: the pairwise fp32 path
    (2, 1024, 4, 1.0),
])
def test_kda_matches_recurrence(B, T, H, g_scale):
    say(f"kda case B{B} T{T} H{H} g_scale{g_scale}")
    q, k, v, gl, beta = _inputs(B, T, H, seed=T + H, g_scale=g_scale)
    o_ref, S_ref = oracle.kda_recurrent(q, k, v, gl, beta)
    o, S = chunk_kda(q.cuda(), k.cuda(), v.cuda(), gl.cuda(), beta.cuda(), output_final_state=True,
                     use_qk_l2norm_in_kernel=True)
    torch.cuda.synchronize()
    _check(o, S, o_ref, S_ref, "kda")


def test_kda_initial_state_and_split_equivalence():
    """Running [0, T1) then [T1, T) with the carried state equals one run (reference tests/test_attention_kimi.py:195-219)."""
    B, T, H, T1 = 1, 320, 2, 128
    q, k, v, gl, beta = (t.cuda() for t in _inputs(B, T, H, seed=5))
    o_full, S_full = chunk_kda(q, k, v, gl, beta, output_final_state=True, use_qk_l2norm_in_kernel=True)
    o1, S1 = chunk_kda(q[:, :T1], k[:, :T1], v[:, :T1], gl[:, :T1], beta[:, :T1], output_final_state=True,
                       use_qk_l2norm_in_kernel=True)
    o2, S2 = chunk_kda(q[:, T1:], k[:, T1:], v[:, T1:], gl[:, T1:], beta[:, T1:], initial_state=S1,
                       output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert_close_bf16(torch.cat([o1, o2], 1), o_full.float(), "split o", max_abs=1e-3, mean_abs=1e-4)
    assert ((S2 - S_full).norm() / S_full.norm()).item() < 1e-5
    # against the oracle with a random initial state
    S0 = torch.randn(B, H, 128, 128, generator=torch.Generator().manual_seed(1)) * 0.1
    o_ref, S_ref = oracle.kda_recurrent(q.cpu(), k.cpu(), v.cpu(), gl.cpu(), beta.cpu(), initial_state=S0)
    o, S = chunk_kda(q, k, v, gl, beta, initial_state=S0.cuda(), output_final_state=True, use_qk_l2norm_in_kernel=True)
    _check(o, S, o_ref, S_ref, "kda with S0")


def test_kda_without_l2norm_and_explicit_scale_bf16_gate():
    B, T, H = 1, 192, 2
    q, k, v, gl, beta = _inputs(B, T, H, seed=9)
    glb = gl.bfloat16()
    o_ref, S_ref = oracle.kda_recurrent(q, k, v, glb.float(), beta, scale=0.25, use_qk_l2norm=False)
    o, S = chunk_kda(q.cuda(), k.cuda(), v.cuda(), glb.cuda(), beta.cuda(), scale=0.25, output_final_state=True,
                     use_qk_l2norm_in_kernel=False)
    _check(o, S, o_ref, S_ref, "kda no-l2norm")


def test_kda_closed_forms():
    """beta = 0: the state only decays and o reads the decayed S0; g = 0, beta = 1, q = k: o = scale * v."""
    B, T, H = 1, 64, 1
    q, k, v, gl, beta = (t.cuda() for t in _inputs(B, T, H, seed=2))
    S0 = torch.randn(B, H, 128, 128, generator=torch.Generator().manual_seed(3)).cuda()
    o, S = chunk_kda(q, k, v, gl, torch.zeros_like(beta), initial_state=S0, output_final_state=True, use_qk_l2norm_in_kernel=True)
    want = S0 * torch.exp(gl.sum(1))[..., None]
    assert ((S - want).norm() / want.norm()).item() < 1e-5
    o2, _ = chunk_kda(k, k, v, torch.zeros_like(gl), torch.ones_like(beta), scale=1.0, output_final_state=False,
                      use_qk_l2norm_in_kernel=True)
    assert_close_bf16(o2, v.float(), "delta rule returns v")


def test_kda_gate_matches_oracle():
    g = torch.Generator().manual_seed(4)
    H, Dk = 4, 128
    x = torch.randn(2, 50, H * Dk, generator=g) * 8
    A_log = torch.log(torch.empty(H).uniform_(1, 16, generator=g))
    bias = torch.randn(H * Dk, generator=g)
    for dt in (torch.float32, torch.bfloat16):
        want = oracle.kda_gate(x.to(dt), A_log.view(1, 1, H, 1), Dk, bias)
        got = fused_kda_gate(x.to(dt).cuda(), A_log.view(1, 1, H, 1).cuda(), Dk, bias.cuda())
        assert got.shape == (2, 50, H, Dk) and got.dtype == dt
        tol = 1e-5 if dt == torch.float32 else 2 ** -7
        assert torch.allclose(got.float().cpu(), want.float(), rtol=tol, atol=1e-6)
    y, b = fused_kda_gate(x.cuda(), A_log.cuda(), Dk, None, b=torch.zeros(2, 50, H).cuda())
    assert torch.allclose(b, torch.full_like(b, 0.5))


def test_kda_rejects_unsupported_shapes():
    z = torch.zeros(1, 64, 1, 136, dtype=torch.bfloat16, device="cuda:0")
    with pytest.raises(RuntimeError, match="Dk"):
        ops.kda_chunk_fwd(z, z, z, z.float(), torch.zeros(1, 64, 1, device="cuda:0"))


def _inputs_dims(B, T, H, Dk, Dv, seed, g_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, T, H, Dk, generator=g), dim=-1).bfloat16()
    k = F.normalize(torch.randn(B, T, H, Dk, generator=g), dim=-1).bfloat16()
    v = torch.randn(B, T, H, Dv, generator=g).bfloat16()
    gl = F.logsigmoid(torch.randn(B, T, H, Dk, generator=g)) * g_scale
    beta = torch.sigmoid(torch.randn(B, T, H, generator=g))
    S0 = torch.randn(B, H, Dk, Dv, generator=g) * 0.1
    return q, k, v, gl, beta, S0


# Head widths other than 128 x 128: the reference's own KDA spec has head_dim 64 (model_specs/old/daisy_pico_linear.yml:5-13)
# and the layer has expand_v (models/daisy/attention_kimi.py:68,80: head_v_dim = head_dim * expand_v).
HEAD_DIMS = [(64, 64), (64, 128), (128, 256), (128, 64), (32, 40), (96, 136), (8, 8), (128, 392)]


@pytest.mark.parametrize("Dk,Dv", HEAD_DIMS)
@pytest.mark.parametrize("T,g_scale,g_bf16", [(200, 1.0, False), (70, 8.0, True)])
def test_kda_other_head_widths_match_recurrence(Dk, Dv, T, g_scale, g_bf16):
    """Chunked and token-by-token kernels, with an initial state, default scale Dk**-0.5, against the recurrence."""
    B, H = 2, 3
    say(f"kda widths Dk{Dk} Dv{Dv} T{T} g_scale{g_scale} g_bf16={g_bf16}")
    q, k, v, gl, beta, S0 = _inputs_dims(B, T, H, Dk, Dv, seed=Dk + Dv + T, g_scale=g_scale)
    if g_bf16:
        gl = gl.bfloat16()
    o_ref, S_ref = oracle.kda_recurrent(q, k, v, gl.float(), beta, initial_state=S0)
    dev = lambda t: t.cuda()
    o, S = chunk_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), initial_state=dev(S0), output_final_state=True,
                     use_qk_l2norm_in_kernel=True)
    assert o.shape == (B, T, H, Dv) and S.shape == (B, H, Dk, Dv)
    _check(o, S, o_ref, S_ref, f"chunked Dk{Dk} Dv{Dv}")
    o_r, S_r = fused_recurrent_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), initial_state=dev(S0), output_final_state=True,
                                   use_qk_l2norm_in_kernel=True)
    _check(o_r, S_r, o_ref, S_ref, f"recurrent Dk{Dk} Dv{Dv}")
    # no initial state, no L2 norm, explicit scale
    o_ref2, S_ref2 = oracle.kda_recurrent(q, k, v, gl.float(), beta, scale=0.3, use_qk_l2norm=False)
    o2, S2 = chunk_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), scale=0.3, output_final_state=True, use_qk_l2norm_in_kernel=False)
    _check(o2, S2, o_ref2, S_ref2, f"chunked, no norm, Dk{Dk} Dv{Dv}")


def test_kda_narrow_heads_decode_steps_and_packed_sequences():
    """Dk = Dv = 64: a chunked prefill continued by in-place decode steps equals one run; packed sequences
    (cu_seqlens) run each from its own state, in both kernels."""
    B, T0, n_steps, H, D = 2, 130, 12, 2, 64
    T = T0 + n_steps
    q, k, v, gl, beta, _ = (t.cuda() for t in _inputs_dims(B, T, H, D, D, seed=5))
    o_ref, S_ref = oracle.kda_recurrent(q.cpu(), k.cpu(), v.cpu(), gl.cpu(), beta.cpu())
    o0, S = chunk_kda(q[:, :T0], k[:, :T0], v[:, :T0], gl[:, :T0], beta[:, :T0], output_final_state=True, use_qk_l2norm_in_kernel=True)
    outs = [o0]
    for t in range(T0, T):
        o_t, S_t = fused_recurrent_kda(q[:, t:t + 1], k[:, t:t + 1], v[:, t:t + 1], gl[:, t:t + 1], beta[:, t:t + 1],
                                       initial_state=S, use_qk_l2norm_in_kernel=True, inplace_state=True)
        assert S_t.data_ptr() == S.data_ptr()
        outs.append(o_t)
    _check(torch.cat(outs, 1), S, o_ref, S_ref, "narrow heads: prefill + decode steps")
    lens = [70, 0, 64, 9]
    cu = torch.tensor([0, 70, 70, 134, 143], dtype=torch.int32)
    q, k, v, gl, beta, _ = _inputs_dims(1, 143, H, D, 2 * D, seed=6)
    S0 = torch.randn(len(lens), H, D, 2 * D, generator=torch.Generator().manual_seed(7)) * 0.1
    dev = lambda t: t.cuda()
    o, S = chunk_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), initial_state=dev(S0), output_final_state=True,
                     use_qk_l2norm_in_kernel=True, cu_seqlens=cu.cuda())
    o_r, S_r = fused_recurrent_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), initial_state=dev(S0), output_final_state=True,
                                   use_qk_l2norm_in_kernel=True, cu_seqlens=cu.cuda())
    for i, n in enumerate(lens):
        s, e = int(cu[i]), int(cu[i + 1])
        if n == 0:
            assert torch.equal(S[i].cpu(), S0[i]) and torch.equal(S_r[i].cpu(), S0[i])
            continue
        o_ref, S_ref = oracle.kda_recurrent(q[:, s:e], k[:, s:e], v[:, s:e], gl[:, s:e], beta[:, s:e], initial_state=S0[i:i + 1])
        _check(o[:, s:e], S[i:i + 1], o_ref, S_ref, f"narrow heads, chunked, sequence {i}")
        _check(o_r[:, s:e], S_r[i:i + 1], o_ref, S_ref, f"narrow heads, recurrent, sequence {i}")


# ---- token-by-token kernel (decode steps, short prompts) ------------------------------------

@pytest.mark.parametrize("B,T,H,g_scale,g_bf16", [
    (2, 1, 3, 1.0, False),     # one decode step
    (1, 17, 2, 1.0, False),
    (2, 130, 2, 0.05, True),   # slow decay, bf16 gate
    (1, 64, 1, 8.0, False),    # very fast decay
])
def test_kda_recurrent_matches_recurrence(B, T, H, g_scale, g_bf16):
    from daisy_amd import fused_recurrent_kda
    say(f"kda recurrent case B{B} T{T} H{H} g_scale{g_scale} g_bf16={g_bf16}")
    q, k, v, gl, beta = _inputs(B, T, H, seed=100 + T + H, g_scale=g_scale)
    if g_bf16:
        gl = gl.bfloat16()
    S0 = torch.randn(B, H, 128, 128, generator=torch.Generator().manual_seed(9)) * 0.1
    o_ref, S_ref = oracle.kda_recurrent(q, k, v, gl.float(), beta, initial_state=S0)
    o, S = fused_recurrent_kda(q.cuda(), k.cuda(), v.cuda(), gl.cuda(), beta.cuda(), initial_state=S0.cuda(),
                               output_final_state=True, use_qk_l2norm_in_kernel=True)
    torch.cuda.synchronize()
    _check(o, S, o_ref, S_ref, "kda recurrent")
    # no initial state, no final state wanted, no L2 norm (inputs are unit vectors already up to bf16 rounding)
    o_ref2, _ = oracle.kda_recurrent(q, k, v, gl.float(), beta, use_qk_l2norm=False)
    o2, S2 = fused_recurrent_kda(q.cuda(), k.cuda(), v.cuda(), gl.cuda(), beta.cuda())
    assert S2 is None
    assert_close_bf16(o2, o_ref2, "kda recurrent (no state): o")


def test_kda_decode_steps_continue_a_chunked_prefill():
    """Prefill T0 tokens with the chunked kernel, then decode token by token with the state carried in place:
    outputs and final state equal one chunked run over all T tokens."""
    from daisy_amd import fused_recurrent_kda
    B, T0, n_steps, H = 2, 200, 24, 2
    T = T0 + n_steps
    q, k, v, gl, beta = (t.cuda() for t in _inputs(B, T, H, seed=77))
    o_ref, S_ref = oracle.kda_recurrent(q.cpu(), k.cpu(), v.cpu(), gl.cpu(), beta.cpu())
    o0, S = chunk_kda(q[:, :T0], k[:, :T0], v[:, :T0], gl[:, :T0], beta[:, :T0], output_final_state=True,
                      use_qk_l2norm_in_kernel=True)
    outs = [o0]
    ptr = S.data_ptr()
    for t in range(T0, T):
        o_t, S_t = fused_recurrent_kda(q[:, t:t + 1], k[:, t:t + 1], v[:, t:t + 1], gl[:, t:t + 1], beta[:, t:t + 1],
                                       initial_state=S, use_qk_l2norm_in_kernel=True, inplace_state=True)
        assert S_t.data_ptr() == ptr
        outs.append(o_t)
    torch.cuda.synchronize()
    _check(torch.cat(outs, 1), S, o_ref, S_ref, "kda prefill + decode steps")


def test_kda_recurrent_rejects_bad_arguments():
    q, k, v, gl, beta = (t.cuda() for t in _inputs(1, 4, 1, seed=3))
    with pytest.raises(RuntimeError, match="not supported"):
        ops.kda_recurrent_fwd(q[..., :60].contiguous(), k[..., :60].contiguous(), v, gl[..., :60].contiguous(), beta)
    with pytest.raises(ValueError):
        ops.kda_recurrent_fwd(q, k, v, gl, beta, inplace_state=True)


def test_kda_cu_seqlens_packs_independent_sequences():
    """Sequences packed along T with ``cu_seqlens`` (the call of models/daisy/attention_kimi.py:133-134
    passes it): each runs from its own initial state, empty ones included."""
    H = 2
    lens = [100, 64, 0, 136]
    T = sum(lens)
    q, k, v, gl, beta = _inputs(1, T, H, seed=11)
    cu = torch.tensor([0, 100, 164, 164, 300], dtype=torch.int32)
    S0 = torch.randn(len(lens), H, 128, 128, generator=torch.Generator().manual_seed(12)) * 0.1
    o, S = chunk_kda(q.cuda(), k.cuda(), v.cuda(), gl.cuda(), beta.cuda(), initial_state=S0.cuda(),
                     output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu.cuda())
    assert o.shape == (1, T, H, 128) and S.shape == (len(lens), H, 128, 128)
    o_r, S_r = fused_recurrent_kda(q.cuda(), k.cuda(), v.cuda(), gl.cuda(), beta.cuda(), initial_state=S0.cuda(),
                                   output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu.cuda())
    for i, n in enumerate(lens):
        s, e = int(cu[i]), int(cu[i + 1])
        if n == 0:
            assert torch.equal(S[i].cpu(), S0[i]) and torch.equal(S_r[i].cpu(), S0[i])
            continue
        o_ref, S_ref = oracle.kda_recurrent(q[:, s:e], k[:, s:e], v[:, s:e], gl[:, s:e], beta[:, s:e], initial_state=S0[i:i + 1])
        _check(o[:, s:e], S[i:i + 1], o_ref, S_ref, f"chunked, sequence {i}")
        _check(o_r[:, s:e], S_r[i:i + 1], o_ref, S_ref, f"recurrent, sequence {i}")
