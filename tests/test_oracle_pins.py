"""Pins the CPU oracle against things that are NOT the oracle's own formulas:
library routines, closed forms, brute-force loops and invariants.  A plausible
mistake in the oracle (wrong rotation sign, off-by-one window, wrong eps, a
transposed operand) fails at least one test here.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle


# ---- RoPE --------------------------------------------------------------------
def test_rope_table_frequencies_are_half_truncated():
    D = 16
    cos, sin = oracle.rope_tables(D, 8)
    assert cos.shape == (8, D // 2)
    # position 1 angle = frequency; first D/4 are (1/1024)**linspace(0,1,D/4), rest zero
    ang = torch.atan2(sin[1], cos[1])
    want = torch.tensor([(1 / 1024) ** (i / 3) for i in range(4)] + [0.0] * 4)
    assert torch.allclose(ang, want, atol=1e-6)
    assert torch.equal(cos[:, 4:], torch.ones(8, 4)) and torch.equal(sin[:, 4:], torch.zeros(8, 4))


def test_rope_table_small_head_dim_keeps_all_frequencies():
    cos, sin = oracle.rope_tables(2, 4)
    assert cos.shape == (4, 1)
    assert torch.allclose(cos[:, 0], torch.cos(torch.arange(4.0)))  # (1/1024)**0 == 1 rad per position


def test_rope_direction_known_answer():
    # D = 2, one pair (x1, x2) = (1, 0) at angle theta -> (cos, -sin): a CLOCKWISE rotation.
    theta = 0.3
    x = torch.tensor([1.0, 0.0]).view(1, 1, 1, 2)
    y = oracle.apply_rope(x, torch.tensor([[math.cos(theta)]]), torch.tensor([[math.sin(theta)]]))
    assert torch.allclose(y.view(2), torch.tensor([math.cos(theta), -math.sin(theta)]), atol=1e-7)
    x = torch.tensor([0.0, 1.0]).view(1, 1, 1, 2)
    y = oracle.apply_rope(x, torch.tensor([[math.cos(theta)]]), torch.tensor([[math.sin(theta)]]))
    assert torch.allclose(y.view(2), torch.tensor([math.sin(theta), math.cos(theta)]), atol=1e-7)


def test_rope_pairs_channel_i_with_i_plus_half():
    D, T = 8, 5
    cos, sin = oracle.rope_tables(D, T, half_truncate=False)
    x = torch.zeros(1, T, 1, D)
    x[..., 1] = 1.0  # only channel 1 set -> only channels 1 and 1 + D/2 may be non-zero
    y = oracle.apply_rope(x, cos, sin)
    nz = (y.abs() > 0).any(dim=0).any(dim=0).any(dim=0)
    assert nz.tolist() == [False, True, False, False, False, True, False, False]


def test_rope_invariants():
    D, T = 32, 40
    g = torch.Generator().manual_seed(0)
    cos, sin = oracle.rope_tables(D, T)
    q = torch.randn(1, T, 2, D, generator=g)
    k = torch.randn(1, T, 2, D, generator=g)
    qr, kr = oracle.apply_rope(q, cos, sin), oracle.apply_rope(k, cos, sin)
    assert torch.equal(qr[:, 0], q[:, 0])                                    # position 0 is the identity
    assert torch.equal(qr[..., D // 4:D // 2], q[..., D // 4:D // 2])         # zero-frequency channels untouched
    assert torch.equal(qr[..., 3 * D // 4:], q[..., 3 * D // 4:])
    n0 = q[..., :D // 2] ** 2 + q[..., D // 2:] ** 2                          # pair norms preserved
    n1 = qr[..., :D // 2] ** 2 + qr[..., D // 2:] ** 2
    assert torch.allclose(n0, n1, atol=1e-5)
    # <rope(q, m), rope(k, n)> depends on m - n only: same vectors placed at shifted positions
    qq = q[:, :1].expand(1, T, 2, D).contiguous()
    kk = k[:, :1].expand(1, T, 2, D).contiguous()
    a, b = oracle.apply_rope(qq, cos, sin), oracle.apply_rope(kk, cos, sin)
    d1 = (a[:, 7] * b[:, 3]).sum(-1)
    d2 = (a[:, 27] * b[:, 23]).sum(-1)
    assert torch.allclose(d1, d2, atol=1e-4)


# ---- RMS norm ------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_matches_library(dtype):
    x = torch.randn(3, 5, 4, 64, generator=torch.Generator().manual_seed(1)).to(dtype)
    want = F.rms_norm(x, (64,))
    got = oracle.rms_norm(x)
    assert (got.float() - want.float()).abs().max().item() <= 1e-6
    if dtype == torch.bfloat16:
        assert torch.equal(got, want)


def test_rms_norm_default_eps_is_the_fp32_epsilon():
    # Tiny inputs make eps visible: mean(x^2) = 1e-6 is >> fp32 eps but << 2**-7.
    x = torch.full((1, 8), 1e-3)
    for dt in (torch.float32, torch.bfloat16):
        xd = x.to(dt)
        lib = F.rms_norm(xd, (8,)).float()
        assert torch.allclose(oracle.rms_norm(xd).float(), lib, rtol=1e-2)
        assert lib[0, 0].item() > 0.9                    # 1/sqrt(1 + 0.119) = 0.945; with eps = 2**-7 it would be 0.011


# ---- masks ---------------------------------------------------------------------
def _brute_mask(ids, window, eos):
    T = len(ids)
    doc, docs = 0, []
    for t in ids:
        if t == eos:
            doc += 1
        docs.append(doc)
    m = torch.zeros(T, T)
    for q in range(T):
        for k in range(T):
            if k > q or q - k >= window or docs[q] != docs[k]:
                m[q, k] = float("-inf")
    return m


@pytest.mark.parametrize("window", [1, 3, 8, 100])
def test_build_attn_mask_brute_force(window):
    ids = [5, 9, 2, 9, 9, 1, 4, 9, 3, 3, 7]
    want = _brute_mask(ids, window, eos=9)
    got = oracle.build_attn_mask(torch.tensor([ids]), window, 9)[0, 0]
    assert torch.equal(got, want)
    ds = oracle.doc_start_from_ids(torch.tensor(ids), 9)
    assert ds.tolist() == [0, 1, 1, 3, 4, 4, 4, 7, 7, 7, 7]
    assert torch.equal(oracle.window_mask(len(ids), window, ds)[0, 0], want)


# ---- attention -------------------------------------------------------------------
def test_sdpa_matches_library_with_additive_mask():
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(2, 3, 17, 16, generator=g) for _ in range(3))
    ids = torch.randint(0, 4, (1, 17), generator=g)
    mask = oracle.build_attn_mask(ids, 5, 2)
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=0.12)
    assert torch.allclose(oracle.sdpa(q, k, v, mask, 0.12), want, atol=1e-5)
    want_c = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.12)
    assert torch.allclose(oracle.windowed_attention(q, k, v, None, 0.12), want_c, atol=1e-5)


def test_windowed_attention_brute_force_rows():
    g = torch.Generator().manual_seed(3)
    T, D, W = 13, 8, 4
    q, k, v = (torch.randn(1, 1, T, D, generator=g) for _ in range(3))
    got = oracle.windowed_attention(q, k, v, W, 0.12)[0, 0]
    for t in range(T):
        lo = max(0, t + 1 - W)  # W keys including the query itself
        s = (k[0, 0, lo:t + 1] @ q[0, 0, t]) * 0.12
        p = torch.exp(s - s.max()); p = p / p.sum()
        assert torch.allclose(got[t], p @ v[0, 0, lo:t + 1], atol=1e-5)


def test_blockwise_equals_dense():
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(1, 2, 300, 16, generator=g) for _ in range(3))
    ids = torch.randint(0, 9, (300,), generator=g)
    ds = oracle.doc_start_from_ids(ids, 0)
    dense = oracle.windowed_attention(q, k, v, 50, 0.12, ds)
    blk = oracle.windowed_attention_blockwise(q, k, v, 50, 0.12, ds, block=64)
    assert torch.allclose(dense, blk, atol=1e-5)
    rows = torch.tensor([0, 17, 299])
    sub = oracle.windowed_attention_blockwise(q, k, v, 50, 0.12, ds, rows=rows)
    assert torch.allclose(dense[:, :, rows], sub, atol=1e-5)


# ---- module level: T steps == one prefill ---------------------------------------
def _module_inputs(T, dim=16, H=2, D=8, seed=0):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(4, dim, dim, generator=g) * 0.3
    x = torch.randn(1, T, dim, generator=g)
    ve = torch.randn(1, T, H * D, generator=g)
    cos, sin = oracle.rope_tables(D, 64)
    return w, x, ve, cos, sin, H, D


@pytest.mark.parametrize("T,window", [(12, 12), (8, 16), (20, 5), (9, 1)])
def test_steps_equal_prefill(T, window):
    """The invariant the reference tests in tests/test_attention.py:80-146."""
    w, x, ve, cos, sin, H, D = _module_inputs(T)
    y_full, k_full, v_full = oracle.attn_prefill(x, w, H, D, cos, sin, window, ve=ve, g_ve=0.4)
    k_ctx = torch.empty(1, 0, H, D)
    v_ctx = torch.empty(1, 0, H, D)
    ys = []
    for t in range(T):
        y, k, v = oracle.attn_step(x[:, t:t + 1], k_ctx, v_ctx, t, w, H, D, cos, sin, window, ve=ve[:, t:t + 1], g_ve=0.4)
        ys.append(y)
        k_ctx, v_ctx = torch.cat([k_ctx, k], 1), torch.cat([v_ctx, v], 1)
    assert torch.allclose(torch.cat(ys, 1), y_full, rtol=1e-4, atol=1e-4)
    assert torch.allclose(k_ctx.transpose(1, 2), k_full, atol=1e-6)
    assert torch.allclose(v_ctx.transpose(1, 2), v_full, atol=1e-6)


def test_prefill_matches_library_pipeline():
    """Whole layer through library calls only (F.linear, F.rms_norm, SDPA is_causal)."""
    w, x, ve, cos, sin, H, D = _module_inputs(10, seed=5)
    y, k, v = oracle.attn_prefill(x, w, H, D, cos, sin, None)
    qkv = F.linear(x, w[:3].flatten(end_dim=1)).view(1, 10, 3 * H, D)
    q_, k_, v_ = (F.rms_norm(t, (D,)) for t in qkv.chunk(3, dim=-2))

    def rot(t):  # rotation written independently: complex multiply by exp(-i*theta)
        z = torch.complex(t[..., :D // 2], t[..., D // 2:]) * torch.complex(cos[:10], -sin[:10])[None, :, None, :]
        return torch.cat([z.real, z.imag], -1)
    want = F.scaled_dot_product_attention(rot(q_).transpose(1, 2), rot(k_).transpose(1, 2), v_.transpose(1, 2),
                                          is_causal=True, scale=0.12)
    want = F.linear(want.transpose(1, 2).reshape(1, 10, H * D), w[3])
    assert torch.allclose(y, want, atol=1e-5)
    assert torch.allclose(k, rot(k_).transpose(1, 2), atol=1e-6)


# ---- KDA ---------------------------------------------------------------------------
def _kda_inputs(B=1, T=9, H=2, Dk=8, Dv=6, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, Dk, generator=g)
    k = torch.randn(B, T, H, Dk, generator=g)
    v = torch.randn(B, T, H, Dv, generator=g)
    gl = F.logsigmoid(torch.randn(B, T, H, Dk, generator=g))
    beta = torch.sigmoid(torch.randn(B, T, H, generator=g))
    return q, k, v, gl, beta


def test_kda_single_token_closed_form():
    q, k, v, g, beta = _kda_inputs(T=1)
    o, S = oracle.kda_recurrent(q, k, v, g, beta, scale=0.5, use_qk_l2norm=False)
    # S0 = 0: S = beta k v^T, o = scale * beta (q.k) v  (the decay does not matter)
    want_S = beta[:, 0, :, None, None] * k[:, 0, :, :, None] * v[:, 0, :, None, :]
    assert torch.allclose(S, want_S, atol=1e-6)
    want_o = 0.5 * beta[:, 0, :, None] * (q[:, 0] * k[:, 0]).sum(-1, keepdim=True) * v[:, 0]
    assert torch.allclose(o[:, 0], want_o, atol=1e-6)


def test_kda_beta_zero_is_pure_decay():
    q, k, v, g, beta = _kda_inputs(T=5)
    S0 = torch.randn(1, 2, 8, 6, generator=torch.Generator().manual_seed(9))
    o, S = oracle.kda_recurrent(q, k, v, g, torch.zeros_like(beta), scale=1.0, initial_state=S0, use_qk_l2norm=False)
    want = S0 * torch.exp(g.sum(1))[..., None]  # decay acts on the Dk (row) axis
    assert torch.allclose(S, want, atol=1e-6)
    want_o_last = torch.einsum("bhkv,bhk->bhv", want, q[:, -1])
    assert torch.allclose(o[:, -1], want_o_last, atol=1e-5)


def test_kda_delta_rule_overwrites_value():
    # g = 0, beta = 1, unit k: after writing (k, v) the state returns exactly v for query k.
    q, k, v, g, beta = _kda_inputs(T=4)
    o, S = oracle.kda_recurrent(k, k, v, torch.zeros_like(g), torch.ones_like(beta), scale=1.0, use_qk_l2norm=True, l2_eps=0.0)
    assert torch.allclose(o, v, atol=1e-5)


def test_kda_split_with_carried_state():
    q, k, v, g, beta = _kda_inputs(T=11, seed=3)
    o, S = oracle.kda_recurrent(q, k, v, g, beta)
    o1, S1 = oracle.kda_recurrent(q[:, :4], k[:, :4], v[:, :4], g[:, :4], beta[:, :4])
    o2, S2 = oracle.kda_recurrent(q[:, 4:], k[:, 4:], v[:, 4:], g[:, 4:], beta[:, 4:], initial_state=S1)
    assert torch.allclose(torch.cat([o1, o2], 1), o, atol=1e-6) and torch.allclose(S2, S, atol=1e-6)


def test_kda_independent_float64_loop():
    """Scalar Python loops in float64, written from the three-line recurrence."""
    q, k, v, g, beta = _kda_inputs(B=1, T=6, H=1, Dk=4, Dv=3, seed=8)
    o, S = oracle.kda_recurrent(q, k, v, g, beta, scale=0.7, use_qk_l2norm=True, l2_eps=1e-6)
    Dk, Dv = 4, 3
    St = [[0.0] * Dv for _ in range(Dk)]
    for t in range(6):
        qq = [float(a) for a in q[0, t, 0]]; kk = [float(a) for a in k[0, t, 0]]
        nq = math.sqrt(sum(a * a for a in qq) + 1e-6); nk = math.sqrt(sum(a * a for a in kk) + 1e-6)
        qq = [a / nq for a in qq]; kk = [a / nk for a in kk]
        for i in range(Dk):
            for j in range(Dv):
                St[i][j] *= math.exp(float(g[0, t, 0, i]))
        pred = [sum(St[i][j] * kk[i] for i in range(Dk)) for j in range(Dv)]
        for i in range(Dk):
            for j in range(Dv):
                St[i][j] += float(beta[0, t, 0]) * kk[i] * (float(v[0, t, 0, j]) - pred[j])
        ot = [0.7 * sum(St[i][j] * qq[i] for i in range(Dk)) for j in range(Dv)]
        assert torch.allclose(o[0, t, 0], torch.tensor(ot, dtype=torch.float32), atol=1e-5)
    assert torch.allclose(S[0, 0], torch.tensor(St, dtype=torch.float32), atol=1e-5)


def test_kda_gate_closed_form():
    g = torch.tensor([[-30.0, -1.0, 0.0, 2.0, 19.0, 25.0, 40.0, 0.5]])  # H = 2, Dk = 4
    A_log = torch.tensor([0.0, math.log(3.0)])
    bias = torch.tensor([0.0, 0.0, 0.0, 0.0, 1.0, 1.0, 1.0, 1.0])
    out = oracle.kda_gate(g, A_log, 4, bias)
    assert out.shape == (1, 2, 4)
    want = -torch.exp(A_log).view(2, 1) * F.softplus(g.view(2, 4) + bias.view(2, 4), beta=1.0, threshold=20.0)
    assert torch.allclose(out[0], want, atol=1e-6)
    assert out[0, 1, 1].item() == pytest.approx(-3.0 * 26.0)   # linear branch above the threshold
    assert (out <= 0).all()
    # the [1,1,H,1] A_log and per-head bias layouts the reference accepts
    out2 = oracle.kda_gate(g, A_log.view(1, 1, 2, 1), 4, torch.tensor([0.0, 1.0]))
    assert torch.allclose(out2, out)


def test_l2norm_known_answers():
    x = torch.tensor([[3.0, 4.0], [0.0, 0.0], [1e-3, 0.0]])
    y = oracle.l2norm(x, eps=0.0)
    assert torch.allclose(y[0], torch.tensor([0.6, 0.8]), atol=1e-7)
    # the epsilon sits inside the square root: x / sqrt(sum(x^2) + eps)
    y = oracle.l2norm(x, eps=1e-6)
    assert y[1].abs().max().item() == 0.0
    assert y[2, 0].item() == pytest.approx(1e-3 / math.sqrt(1e-6 + 1e-6), rel=1e-5)
    # and it is what kda_recurrent applies to q and k
    q, k, v, g, beta = _kda_inputs(T=3)
    o1, S1 = oracle.kda_recurrent(q, k, v, g, beta, use_qk_l2norm=True, l2_eps=1e-6)
    o2, S2 = oracle.kda_recurrent(oracle.l2norm(q), oracle.l2norm(k), v, g, beta, use_qk_l2norm=False)
    assert torch.allclose(o1, o2, atol=1e-6) and torch.allclose(S1, S2, atol=1e-6)


# ---- value-embedding mix (models/daisy/attention.py:132-135,186-190) --------------------------
def _mix_case(g_ve, T=7, window=4):
    w, x, ve, cos, sin, H, D = _module_inputs(T, seed=11)
    y, k, v = oracle.attn_prefill(x, w, H, D, cos, sin, window, ve=ve, g_ve=g_ve)
    _, _, v_plain = oracle.attn_prefill(x, w, H, D, cos, sin, window)             # no mix: v = norm(v)
    return v, v_plain, ve.view(1, T, H, D).transpose(1, 2), (w, x, ve, cos, sin, H, D, y)


def test_value_embedding_mix_known_answers_in_prefill():
    v, v_plain, ve_, _ = _mix_case(30.0)          # sigmoid(30) = 1 in fp32: v untouched
    assert torch.equal(v, v_plain)
    v, v_plain, ve_, _ = _mix_case(-30.0)         # sigmoid(-30) ~ 1e-13: ve takes over
    assert torch.allclose(v, ve_, atol=1e-6)
    # the reference's first-layer gate logit (attention.py:96): sigmoid(0.3228) = 0.58 by hand
    g = 1.0 / (1.0 + math.exp(-0.3228))
    assert g == pytest.approx(0.58, abs=1e-4)
    v, v_plain, ve_, _ = _mix_case(0.3228)
    assert torch.allclose(v, 0.58 * v_plain + 0.42 * ve_, atol=2e-4)
    assert not torch.allclose(v, 0.42 * v_plain + 0.58 * ve_, atol=1e-2)          # the swapped gate is visibly different


def test_value_embedding_mix_known_answers_in_step():
    T, window = 6, 4
    for g_ve, a, b in ((30.0, 1.0, 0.0), (-30.0, 0.0, 1.0), (0.3228, 0.58, 0.42)):
        w, x, ve, cos, sin, H, D = _module_inputs(T, seed=12)
        k_ctx = torch.randn(1, 3, H, D, generator=torch.Generator().manual_seed(1))
        v_ctx = torch.randn(1, 3, H, D, generator=torch.Generator().manual_seed(2))
        _, _, v_new = oracle.attn_step(x[:, 3:4], k_ctx, v_ctx, 3, w, H, D, cos, sin, window, ve=ve[:, 3:4], g_ve=g_ve)
        _, _, v_plain = oracle.attn_step(x[:, 3:4], k_ctx, v_ctx, 3, w, H, D, cos, sin, window)
        want = a * v_plain + b * ve[:, 3:4].view(1, 1, H, D)
        assert torch.allclose(v_new, want, atol=2e-4), g_ve
        # and the mixed value is what the step attends: with one cached row removed from play
        # (window 1) the output is o_proj(v_new)
        y1, _, v1 = oracle.attn_step(x[:, 3:4], k_ctx, v_ctx, 3, w, H, D, cos, sin, 1, ve=ve[:, 3:4], g_ve=g_ve)
        assert torch.allclose(y1, F.linear(v1.reshape(1, 1, H * D), w[3]), atol=1e-5)


# ---- the KDA layer's neighbours (models/daisy/attention_kimi.py:41-62,90-92,155-158) ----------
def test_short_conv_matches_library_conv_and_silu():
    g = torch.Generator().manual_seed(20)
    B, T, C, K = 2, 19, 6, 4
    x = torch.randn(B, T, C, generator=g)
    w = torch.randn(C, 1, K, generator=g)
    bias = torch.randn(C, generator=g)
    y, cache = oracle.short_conv(x, w, bias, output_final_state=True)
    padded = F.pad(x.transpose(1, 2), (K - 1, 0))                       # K-1 zeros before the sequence
    want = F.silu(F.conv1d(padded, w, bias, groups=C)).transpose(1, 2)
    assert torch.allclose(y, want, atol=1e-5)
    assert torch.equal(cache, x[:, -K:].transpose(1, 2))                # the last K inputs, [B, C, K]
    y_lin, _ = oracle.short_conv(x, w, None, activation=None)
    assert torch.allclose(y_lin, F.conv1d(padded, w, None, groups=C).transpose(1, 2), atol=1e-5)


def test_short_conv_brute_force_taps():
    g = torch.Generator().manual_seed(21)
    T, C, K = 7, 3, 4
    x = torch.randn(1, T, C, generator=g)
    w = torch.randn(C, K, generator=g)
    win = torch.randn(1, C, K, generator=g)
    y, _ = oracle.short_conv(x, w, cache=win, activation=None)
    for t in range(T):
        for c in range(C):
            acc = 0.0
            for j in range(K):
                ti = t - (K - 1) + j                                     # the last tap multiplies the current input
                xin = float(x[0, ti, c]) if ti >= 0 else float(win[0, c, K + ti])
                acc += float(w[c, j]) * xin
            assert y[0, t, c].item() == pytest.approx(acc, abs=1e-5)


def test_short_conv_carried_window_and_packed_sequences():
    g = torch.Generator().manual_seed(22)
    T, C, K = 23, 8, 4
    x = torch.randn(1, T, C, generator=g)
    w = torch.randn(C, 1, K, generator=g)
    whole, cache = oracle.short_conv(x, w, output_final_state=True)
    for cut in (1, 2, 3, 9):                                             # also cuts shorter than the window
        y1, c1 = oracle.short_conv(x[:, :cut], w, output_final_state=True)
        y2, c2 = oracle.short_conv(x[:, cut:], w, cache=c1, output_final_state=True)
        assert torch.allclose(torch.cat([y1, y2], 1), whole, atol=1e-6) and torch.allclose(c2, cache)
    cu = torch.tensor([0, 5, 5, 6, 23])
    packed, caches = oracle.short_conv(x, w, output_final_state=True, cu_seqlens=cu)
    for i in range(4):
        s, e = int(cu[i]), int(cu[i + 1])
        if e > s:
            alone, c = oracle.short_conv(x[:, s:e], w, output_final_state=True)
            assert torch.allclose(packed[:, s:e], alone, atol=1e-6) and torch.allclose(caches[i], c[0])
        else:
            assert caches[i].abs().max().item() == 0.0                   # an empty sequence keeps its (zero) window


def test_gated_rms_norm_matches_library_pieces():
    g = torch.Generator().manual_seed(23)
    x = torch.randn(3, 5, 2, 128, generator=g) * 3
    gate = torch.randn(3, 5, 2, 128, generator=g) * 2
    w = 1 + 0.1 * torch.randn(128, generator=g)
    want = F.rms_norm(x, (128,), w, 1e-5) * torch.sigmoid(gate)
    assert torch.allclose(oracle.gated_rms_norm(x, gate, w, 1e-5), want, atol=1e-5)
    # eps matters for small rows and sits under the mean of squares
    tiny = torch.full((1, 128), 1e-3)
    out = oracle.gated_rms_norm(tiny, torch.zeros(1, 128), torch.ones(128), 1e-5)
    assert out[0, 0].item() == pytest.approx(0.5 * 1e-3 / math.sqrt(1e-6 + 1e-5), rel=1e-5)
