"""KimiLinearSelfAttention drop-in (models/daisy/attention_kimi.py:64-200) on the GPU.

The layer runs on the HIP kernels; here it is checked against the oracle's restatement of the
layer (oracle/kimi.py: fp32 short convolutions, gate, naive recurrence, gated norm; the projections as
library GEMMs on the CPU), and against itself: prompt + single-token steps must equal one full
forward (the property the reference's tests/test_attention_kimi.py:161-219 checks with tolerances
2e-2 / 3e-2).  The streaming kernels (short convolution, gated norm) and the packed-sequence
(cu_seqlens) forms of all kernels are checked against the oracle one by one.
"""
import pytest
import torch
import torch.nn.functional as F

import oracle
from daisy_amd import KimiLinearSelfAttention
from helpers import say

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _layer(dim=256, H=2, seed=0, receives_ve=False, head_dim=128, expand_v=1.0, conv_size=4):
    torch.manual_seed(seed)
    m = KimiLinearSelfAttention(dim, H, max_seq_len=1024, head_dim=head_dim, expand_v=expand_v, conv_size=conv_size,
                                receives_ve=receives_ve)
    with torch.no_grad():
        for p in m.parameters():
            if p.dim() >= 2 and p.dtype == torch.bfloat16:
                p.copy_((torch.randn(p.shape) * (0.5 / p.shape[-1] ** 0.5)).bfloat16())
        m.dt_bias.copy_(torch.randn(m.dt_bias.shape) * 0.5)
        m.o_norm.weight.copy_((1 + 0.1 * torch.randn(m.o_norm.weight.shape)).bfloat16())
    return m.eval()


def _cpu_reference(m, x, ve=None, cu_seqlens=None):
    """The oracle's layer on the parameters of ``m`` (a CPU copy of the module, used as a parameter store only)."""
    params = {k: v.detach() for k, v in m.state_dict().items()}
    g_ve = float(m.g_ve) if m.receives_ve else None
    return oracle.kimi_layer_forward(x, params, m.num_heads, m.head_k_dim, ve=ve, g_ve=g_ve, cu_seqlens=cu_seqlens)


def _close(a, b, what, tol):
    err = (a.float().cpu() - b.float().cpu()).abs()
    say(f"{what}: max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e}")
    assert err.max().item() <= tol, what


@pytest.mark.parametrize("B,T,receives_ve", [(1, 200, False), (2, 96, True)])
def test_forward_matches_cpu_layer(B, T, receives_ve):
    with torch.no_grad():
        m = _layer(receives_ve=receives_ve)
        g = torch.Generator().manual_seed(1)
        x = torch.randn(B, T, 256, generator=g).bfloat16()
        ve = torch.randn(B, T, 256, generator=g).bfloat16() if receives_ve else None
        y_ref = _cpu_reference(m, x, ve)
        md = _layer(receives_ve=receives_ve).to(DEV)
        md.load_state_dict(m.state_dict())
        y = md(x.to(DEV), None if ve is None else ve.to(DEV))
        assert y.shape == (B, T, 256) and y.dtype == torch.bfloat16
        _close(y, y_ref, "forward vs CPU layer", 3e-2)


@pytest.mark.parametrize("H,head_dim,expand_v,conv_size", [
    (4, 64, 1.0, 4),      # the reference's own KDA spec: head_dim 64 (model_specs/old/daisy_pico_linear.yml:5-13)
    (4, 64, 2.0, 3),      # value heads twice as wide as key heads (attention_kimi.py:68,80)
    (2, 128, 2.0, 4),     # 256 value columns per head: two passes of the delta-rule kernels
    (8, 32, 1.0, 2),
])
def test_other_head_widths_match_cpu_layer_and_stream(H, head_dim, expand_v, conv_size):
    """Forward against the oracle's layer, and prompt + decode steps against the full forward, at head widths
    other than 128."""
    with torch.no_grad():
        kw = dict(H=H, head_dim=head_dim, expand_v=expand_v, conv_size=conv_size, seed=7)
        m = _layer(**kw)
        assert m.head_v_dim == int(head_dim * expand_v) and m.value_dim == H * m.head_v_dim
        g = torch.Generator().manual_seed(8)
        x = torch.randn(2, 150, 256, generator=g).bfloat16()
        params = {k: v.detach() for k, v in m.state_dict().items()}
        y_ref = oracle.kimi_layer_forward(x, params, H, head_dim, conv_size=conv_size)
        md = _layer(**kw).to(DEV)
        md.load_state_dict(m.state_dict())
        xd = x.to(DEV)
        y = md(xd, None)
        _close(y, y_ref, f"forward vs CPU layer, head_dim {head_dim} expand_v {expand_v}", 3e-2)
        y0, _, _ = md.prefill(xd[:, :130], None)
        ys = [y0] + [md.step(xd[:, t:t + 1], None, None, t, None, None)[0] for t in range(130, 150)]
        _close(torch.cat(ys, 1), y, "prefill + steps vs full forward", 2e-2)


def test_constructor_refuses_what_the_kernels_do_not_serve():
    for kw in (dict(head_dim=160), dict(head_dim=36), dict(head_dim=128, expand_v=0.75), dict(head_dim=128, conv_size=5)):
        with pytest.raises(ValueError, match="not supported"):
            KimiLinearSelfAttention(256, 2, max_seq_len=64, **kw)


def test_prefill_then_steps_equals_full_forward():
    with torch.no_grad():
        m = _layer(seed=2).to(DEV)
        T0, n_steps = 150, 40
        x = torch.randn(2, T0 + n_steps, 256, generator=torch.Generator().manual_seed(3)).bfloat16().to(DEV)
        y_full = m(x, None)
        assert m._recurrent_state is None, "forward must not leave a state behind"
        y0, k, v = m.prefill(x[:, :T0], None, attn_mask=None)
        assert k is None and v is None
        ys = [y0]
        state_ptr = None
        for t in range(T0, T0 + n_steps):
            y, _, _ = m.step(x[:, t:t + 1], None, None, t, None, window=None)
            ys.append(y)
            if state_ptr is None:
                state_ptr = m._recurrent_state.data_ptr()
            assert m._recurrent_state.data_ptr() == state_ptr, "decode steps update the state in place"
        _close(torch.cat(ys, 1), y_full, "prefill + steps vs full forward", 2e-2)
        assert m._seen == T0 + n_steps
        m.reset_history()
        assert m._recurrent_state is None and m._conv_state is None and m._seen == 0
        # token-by-token from the start (no prefill) equals the full forward too
        ys = [m.step(x[:, t:t + 1], None, None, t, None, window=None)[0] for t in range(24)]
        _close(torch.cat(ys, 1), y_full[:, :24], "streaming from an empty state", 2e-2)


def test_parameter_names_and_dtypes_follow_the_reference():
    m = KimiLinearSelfAttention(256, 2, 64, 128).bfloat16()
    keys = set(m.state_dict().keys())
    for k in ("q_proj.weight", "k_proj.weight", "v_proj.weight", "q_conv1d.weight", "k_conv1d.weight", "v_conv1d.weight",
              "f_proj.0.weight", "f_proj.1.weight", "b_proj.weight", "A_log", "dt_bias", "g_proj.0.weight",
              "g_proj.1.weight", "g_proj.1.bias", "o_norm.weight", "o_proj.weight"):
        assert k in keys, k
    assert m.A_log.shape == (1, 1, 2, 1) and m.A_log.dtype == torch.float32 and m.dt_bias.dtype == torch.float32
    assert m.q_conv1d.weight.shape == (256, 1, 4)
    with pytest.raises(AssertionError):
        m.to(DEV)(torch.zeros(1, 4, 256, device=DEV, dtype=torch.bfloat16), None, block_mask=object())


def test_padding_mask_packs_sequences():
    """A [B, S] padding mask (models/daisy/attention_kimi.py:150-154): every row runs as its own
    sequence on its tokens only, padded positions come back as zeros."""
    with torch.no_grad():
        m = _layer(seed=4).to(DEV)
        B, S = 3, 160
        x = torch.randn(B, S, 256, generator=torch.Generator().manual_seed(5)).bfloat16().to(DEV)
        lens = [160, 97, 1]
        mask = torch.zeros(B, S, dtype=torch.int32)
        for b, n in enumerate(lens):
            mask[b, S - n:] = 1          # left padding
        y = m(x, None, attn_mask=mask.to(DEV))
        assert y.shape == (B, S, 256)
        for b, n in enumerate(lens):
            y_b = m(x[b:b + 1, S - n:], None)
            _close(y[b, S - n:], y_b[0], f"row {b} ({n} tokens) vs the row alone", 2e-2)
            assert not y[b, :S - n].any(), "padded positions must be zero"
        # with a state: prefill on the padded batch, then a step, equals the rows one by one
        m.reset_history()
        m.prefill(x, None, attn_mask=mask.to(DEV))
        assert m._recurrent_state.shape[0] == B
        x1 = torch.randn(B, 1, 256, generator=torch.Generator().manual_seed(6)).bfloat16().to(DEV)
        y1, _, _ = m.step(x1, None, None, S, None, None)
        for b, n in enumerate(lens):
            m.reset_history()
            m.prefill(x[b:b + 1, S - n:], None)
            y1_b, _, _ = m.step(x1[b:b + 1], None, None, n, None, None)
            _close(y1[b], y1_b[0], f"step after padded prefill, row {b}", 2e-2)


@pytest.mark.parametrize("B,T,C,K,bias,with_cache", [(2, 70, 256, 4, False, False), (1, 1, 64, 4, True, True),
                                                     (3, 33, 128, 3, True, True), (1, 200, 2048, 4, False, True),
                                                     (2, 2, 64, 2, False, True)])
def test_short_convolution_kernel_matches_oracle(B, T, C, K, bias, with_cache):
    """The streaming kernel against oracle.short_conv (fp32 taps + SiLU on the same bf16 inputs)."""
    from daisy_amd import ops
    g = torch.Generator().manual_seed(T + C)
    w = (torch.randn(C, 1, K, generator=g) * 0.4).bfloat16()
    bs = (torch.randn(C, generator=g) * 0.3).bfloat16() if bias else None
    x = torch.randn(B, T, C, generator=g).bfloat16()
    cache = torch.randn(B, C, K, generator=g).bfloat16() if with_cache else None
    y_ref, c_ref = oracle.short_conv(x, w, bs, cache, output_final_state=True)
    pre_ref, _ = oracle.short_conv(x, w, bs, cache, activation=None)
    dev = lambda t: None if t is None else t.to(DEV)
    y, c = ops.short_conv(dev(x), dev(w), dev(bs), dev(cache), True)
    assert y.shape == (B, T, C) and c.shape == (B, C, K) and y.dtype == torch.bfloat16
    assert torch.equal(c.cpu().float(), c_ref), "carried window differs"
    # the kernel rounds the pre-activation to bf16, applies SiLU and rounds again: two bf16 roundings
    # of values of the pre-activation's size against the unrounded oracle
    err = (y.float().cpu() - y_ref).abs()
    tol = 2.0 ** -7 * pre_ref.abs().clamp_min(0.25)
    say(f"short conv B{B} T{T} C{C} K{K}: max-abs {err.max().item():.3e}")
    assert bool((err <= tol).all())
    # a sequence cut in two with the window carried equals the sequence in one go
    if T >= 2:
        h = T // 2
        y1, c1 = ops.short_conv(dev(x[:, :h]), dev(w), dev(bs), dev(cache), True)
        y2, c2 = ops.short_conv(dev(x[:, h:]), dev(w), dev(bs), c1, True)
        assert torch.equal(torch.cat([y1, y2], dim=1), y) and torch.equal(c2, c)


@pytest.mark.parametrize("K,bias,with_cache", [(4, False, False), (4, True, True), (3, False, True), (2, True, False)])
def test_short_convolution_over_packed_sequences_matches_oracle(K, bias, with_cache):
    """cu_seqlens read on the device: ragged sequences (one empty, some shorter than the window, boundaries
    inside and at the edges of the kernel's 32-step segments) against the oracle's per-sequence loop."""
    from daisy_amd import ops
    g = torch.Generator().manual_seed(40 + K)
    C = 136
    lens = [5, 0, 1, 31, 32, 33, 2, 64, 70, 3]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    T, N = int(cu[-1]), len(lens)
    x = torch.randn(1, T, C, generator=g).bfloat16()
    w = (torch.randn(C, 1, K, generator=g) * 0.4).bfloat16()
    bs = (torch.randn(C, generator=g) * 0.3).bfloat16() if bias else None
    cache = torch.randn(N, C, K, generator=g).bfloat16() if with_cache else None
    y_ref, c_ref = oracle.short_conv(x, w, bs, cache, output_final_state=True, cu_seqlens=cu)
    pre_ref, _ = oracle.short_conv(x, w, bs, cache, cu_seqlens=cu, activation=None)
    dev = lambda t: None if t is None else t.to(DEV)
    y, c = ops.short_conv(dev(x), dev(w), dev(bs), dev(cache), True, cu_seqlens=cu.to(DEV))
    assert c.shape == (N, C, K)
    assert torch.equal(c.cpu().float(), c_ref), "carried windows differ"
    err = (y.float().cpu() - y_ref).abs()
    assert bool((err <= 2.0 ** -7 * pre_ref.abs().clamp_min(0.25)).all()), err.max().item()
    # each sequence alone through the plain kernel gives the same bits
    for i in range(N):
        s, e = int(cu[i]), int(cu[i + 1])
        if e > s:
            y_i, c_i = ops.short_conv(dev(x[:, s:e]), dev(w), dev(bs), None if cache is None else dev(cache[i:i + 1]), True)
            assert torch.equal(y_i, y[:, s:e]) and torch.equal(c_i[0], c[i]), f"sequence {i}"


def test_short_convolution_window_updated_in_place():
    """Decode steps shift the window inside the cache tensor: same outputs and same window as the
    out-of-place call, for one step and for a few steps at once; long inputs are refused."""
    from daisy_amd import ops
    g = torch.Generator().manual_seed(12)
    B, C = 3, 256
    for K in (4, 3, 2):
        w = (torch.randn(C, 1, K, generator=g) * 0.3).bfloat16().to(DEV)
        bias = (torch.randn(C, generator=g) * 0.1).bfloat16().to(DEV)
        window = torch.randn(B, C, K, generator=g).bfloat16().to(DEV)
        for T in (1, 1, 2, 5, 32):
            x = torch.randn(B, T, C, generator=g).bfloat16().to(DEV)
            y_ref, w_ref = ops.short_conv(x, w, bias, window, True)
            mine = window.clone()
            y, w_new = ops.short_conv(x, w, bias, mine, True, inplace_cache=True)
            assert w_new.data_ptr() == mine.data_ptr()
            assert torch.equal(y, y_ref) and torch.equal(mine, w_ref), f"K={K} T={T}"
            window = w_ref
    with pytest.raises(RuntimeError, match="in place"):
        ops.short_conv(torch.zeros(B, 40, C, device=DEV, dtype=torch.bfloat16), w, bias, window.clone(), True, inplace_cache=True)


@pytest.mark.parametrize("rows,D", [(5, 128), (1000, 128), (77, 64), (33, 32), (130, 256)])
def test_gated_rmsnorm_kernel_matches_oracle(rows, D):
    from daisy_amd import ops
    g = torch.Generator().manual_seed(rows)
    w = (1 + 0.2 * torch.randn(D, generator=g)).bfloat16()
    x, gate = torch.randn(rows, D, generator=g).bfloat16() * 3, torch.randn(rows, D, generator=g).bfloat16() * 2
    ref = oracle.gated_rms_norm(x, gate, w, 1e-5)
    out = ops.gated_rmsnorm(x.to(DEV), gate.to(DEV), w.to(DEV), 1e-5)
    err = (out.float().cpu() - ref).abs()
    say(f"gated norm rows{rows} D{D}: max-abs {err.max().item():.3e}")
    assert bool((err <= 2.0 ** -7 * ref.abs().clamp_min(1e-3)).all())      # one bf16 rounding of the result


def test_layer_ops_refuse_cpu_tensors():
    """One path: the layer's streaming ops raise for CPU tensors like every other op of the package."""
    from daisy_amd.attention_kimi import GatedRMSNorm, ShortConvolution
    with pytest.raises(RuntimeError, match="no CPU path"):
        ShortConvolution(64, 4)(torch.zeros(1, 8, 64, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="no CPU path"):
        GatedRMSNorm(128)(torch.zeros(4, 128, dtype=torch.bfloat16), torch.zeros(4, 128, dtype=torch.bfloat16))


def _kda_pack(lens, H=2, seed=0):
    g = torch.Generator().manual_seed(seed)
    T = sum(lens)
    q = torch.randn(1, T, H, 128, generator=g).bfloat16()
    k = torch.randn(1, T, H, 128, generator=g).bfloat16()
    v = torch.randn(1, T, H, 128, generator=g).bfloat16()
    gl = F.logsigmoid(torch.randn(1, T, H, 128, generator=g))
    beta = torch.sigmoid(torch.randn(1, T, H, generator=g))
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    return q, k, v, gl, beta, cu


@pytest.mark.parametrize("lens,with_state", [([200, 64, 1, 0, 130], True), ([63, 65], False), ([5], True),
                                             ([0, 0, 70, 0], True), ([128, 128, 128], False)])
def test_chunk_kda_over_packed_sequences_matches_oracle(lens, with_state):
    """daisy_kda_chunk_varlen_fwd: the sequence boundaries are read by the kernels (no host loop, no
    synchronisation); every sequence against the oracle's recurrence on its own slice."""
    from daisy_amd import chunk_kda
    q, k, v, gl, beta, cu = _kda_pack(lens, seed=len(lens))
    N, H = len(lens), q.shape[2]
    S0 = torch.randn(N, H, 128, 128, generator=torch.Generator().manual_seed(9)) * 0.1 if with_state else None
    dev = lambda t: None if t is None else t.to(DEV)
    o, S = chunk_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), initial_state=dev(S0), output_final_state=True,
                     use_qk_l2norm_in_kernel=True, cu_seqlens=cu.to(DEV))
    assert o.shape == q.shape and S.shape == (N, H, 128, 128)
    for i in range(N):
        s, e = int(cu[i]), int(cu[i + 1])
        s0 = None if S0 is None else S0[i:i + 1]
        if e == s:
            want = s0 if s0 is not None else torch.zeros(1, H, 128, 128)
            assert torch.equal(S[i:i + 1].cpu(), want), f"an empty sequence ({i}) must keep its state"
            continue
        o_ref, S_ref = oracle.kda_recurrent(q[:, s:e], k[:, s:e], v[:, s:e], gl[:, s:e], beta[:, s:e], initial_state=s0)
        err = (o[:, s:e].float().cpu() - o_ref).abs()
        assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3, (i, err.max().item())
        rel = ((S[i:i + 1].cpu() - S_ref).norm() / S_ref.norm()).item()
        assert rel <= 1e-3, (i, rel)


def test_fused_recurrent_kda_over_packed_sequences_matches_oracle():
    from daisy_amd import fused_recurrent_kda
    lens = [7, 0, 1, 20]
    q, k, v, gl, beta, cu = _kda_pack(lens, seed=5)
    N, H = len(lens), q.shape[2]
    S0 = torch.randn(N, H, 128, 128, generator=torch.Generator().manual_seed(3)) * 0.1
    dev = lambda t: t.to(DEV)
    o, S = fused_recurrent_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), initial_state=dev(S0), output_final_state=True,
                               use_qk_l2norm_in_kernel=True, cu_seqlens=cu.to(DEV))
    for i in range(N):
        s, e = int(cu[i]), int(cu[i + 1])
        o_ref, S_ref = oracle.kda_recurrent(q[:, s:e], k[:, s:e], v[:, s:e], gl[:, s:e], beta[:, s:e], initial_state=S0[i:i + 1])
        if e > s:
            assert (o[:, s:e].float().cpu() - o_ref).abs().max().item() <= 2e-2
        assert ((S[i:i + 1].cpu() - S_ref).norm() / S_ref.norm()).item() <= 1e-3


def test_packed_bounds_that_break_the_contract_stay_inside_the_tensors():
    """Bounds are forced into 0..T and made non-decreasing on the device: nonsense in, no fault out."""
    from daisy_amd import chunk_kda
    q, k, v, gl, beta, _ = _kda_pack([150], seed=8)
    bad = torch.tensor([5, -3, 90, 40, 10 ** 6], dtype=torch.int32)      # reads as 0, 5, 90, 90, 150 (running maximum)
    dev = lambda t: t.to(DEV)
    o, S = chunk_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), output_final_state=True, use_qk_l2norm_in_kernel=True,
                     cu_seqlens=bad.to(DEV))
    good = torch.tensor([0, 5, 90, 90, 150], dtype=torch.int32)
    o2, S2 = chunk_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), output_final_state=True, use_qk_l2norm_in_kernel=True,
                       cu_seqlens=good.to(DEV))
    assert torch.equal(o, o2) and torch.equal(S, S2) and bool(torch.isfinite(o.float()).all())


def test_bounds_outside_the_token_range_are_clamped_the_same_way_by_every_packed_kernel():
    """Every packed-sequence kernel forces each bound into 0..T (the one rule they share): bounds that are ordered
    but reach outside the token range give exactly what the clamped bounds give -- in the chunked and the
    token-by-token delta rule and in the short convolution.  Bounds that are out of order break the contract; each
    kernel then stays inside the tensors and leaves finite states, but which tokens it assigns to which sequence is
    left open (the header says so)."""
    from daisy_amd import chunk_kda, fused_recurrent_kda, ops
    T, C, K = 150, 64, 4
    q, k, v, gl, beta, _ = _kda_pack([T], seed=8)
    dev = lambda t: t.to(DEV)
    wide = torch.tensor([-7, 5, 90, 10 ** 6], dtype=torch.int32).to(DEV)
    clamped = torch.tensor([0, 5, 90, T], dtype=torch.int32).to(DEV)
    broken = torch.tensor([5, -3, 90, 40, 10 ** 6], dtype=torch.int32).to(DEV)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, T, C, generator=g).bfloat16().to(DEV)
    w = (torch.randn(C, K, generator=g) * 0.5).bfloat16().to(DEV)
    win = torch.randn(3, C, K, generator=g).bfloat16().to(DEV)

    def run_all(cu, n):
        out = {}
        out["chunk"] = chunk_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), output_final_state=True,
                                 use_qk_l2norm_in_kernel=True, cu_seqlens=cu)
        out["recurrent"] = fused_recurrent_kda(dev(q), dev(k), dev(v), dev(gl), dev(beta), output_final_state=True,
                                               use_qk_l2norm_in_kernel=True, cu_seqlens=cu)
        cache = win if n == 3 else torch.zeros(n, C, K, dtype=torch.bfloat16, device=DEV)
        out["conv"] = ops.short_conv(x, w, cache=cache, output_final_state=True, cu_seqlens=cu)
        torch.cuda.synchronize()
        return out

    a, b = run_all(wide, 3), run_all(clamped, 3)
    for name in a:
        assert torch.equal(a[name][0], b[name][0]), f"{name}: outputs differ between wide and clamped bounds"
        assert torch.equal(a[name][1], b[name][1]), f"{name}: states / windows differ between wide and clamped bounds"
    c = run_all(broken, 4)
    # Rows (and convolution windows) that end up in no sequence are left unwritten, so only the delta-rule states are
    # looked at; for the convolution the point is that the launch completes (run_all synchronises).
    for name in ("chunk", "recurrent"):
        assert bool(torch.isfinite(c[name][1].float()).all()), f"{name}: state with out-of-order bounds"


@pytest.mark.parametrize("B", [1, 3])
def test_stacked_input_projections_equal_the_separate_ones(B):
    """A decode step of a few sequences reads the six projections of the layer's input through one stacked matrix
    (models/daisy/attention_kimi.py:99-118 are six separate Linear modules): every output equals the separate
    launch's bit for bit, the stack follows a weight that changes, and a stale stack is not rebuilt under capture."""
    from daisy_amd.attention_kimi import _project
    with torch.no_grad():
        m = _layer(seed=11).to(DEV)
        g = torch.Generator().manual_seed(12)
        x = torch.randn(B, 1, 256, generator=g).bfloat16().to(DEV)
        lins = (m.q_proj, m.k_proj, m.v_proj, m.f_proj[0], m.g_proj[0], m.b_proj)

        def separate():
            return tuple(_project(l, x) for l in lins)

        got = m._input_projections(x)
        assert m._stacked_w is not None and m._stacked_w.shape[0] % 8 == 0
        assert m._stacked_w.shape[0] >= sum(l.weight.shape[0] for l in lins)
        for a, b in zip(got, separate()):
            assert a.shape == b.shape and torch.equal(a, b)
        m.k_proj.weight.mul_(1.5)                        # in place: same address, new version
        for a, b in zip(m._input_projections(x), separate()):
            assert torch.equal(a, b)
        # the whole step through the stacked matrix equals the step through the separate launches
        xs = torch.randn(B, 6, 256, generator=g).bfloat16().to(DEV)
        m.reset_history()
        m.prefill(xs[:, :3], None, attn_mask=None)
        y_stacked = [m.step(xs[:, t:t + 1], None, None, t, None, window=None)[0] for t in range(3, 6)]
        m.reset_history()
        m._input_projections = lambda inp: tuple(_project(l, inp) for l in lins)
        m.prefill(xs[:, :3], None, attn_mask=None)
        y_separate = [m.step(xs[:, t:t + 1], None, None, t, None, window=None)[0] for t in range(3, 6)]
        del m._input_projections
        for a, b in zip(y_stacked, y_separate):
            assert torch.equal(a, b)
        # more rows than the few-rows kernel is used for: the separate library products
        wide = torch.randn(8, 1, 256, generator=g).bfloat16().to(DEV)
        for a, l in zip(m._input_projections(wide), lins):
            assert torch.equal(a, l(wide))
        # a stack that has gone stale while the stream is capturing is left alone
        m.v_proj.weight.mul_(0.5)
        key_before = m._stacked_key
        graph = torch.cuda.CUDAGraph()
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            with torch.cuda.graph(graph, stream=s):
                captured = m._input_projections(x)
        assert m._stacked_key == key_before
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(captured, separate()):
            assert torch.equal(a, b)
