"""KimiLinearSelfAttention drop-in (models/daisy/attention_kimi.py:64-200) on the GPU.

The layer's delta-rule core runs on the HIP kernels; here it is checked against the same layer
evaluated on the CPU with the oracle's gate and naive fp32 recurrence in place of the kernels, and
against itself: prompt + single-token steps must equal one full forward (the property the
reference's tests/test_attention_kimi.py:161-219 checks with tolerances 2e-2 / 3e-2).
"""
import pytest
import torch
import torch.nn.functional as F

import oracle
from daisy_amd import KimiLinearSelfAttention
from helpers import say

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _layer(dim=256, H=2, seed=0, receives_ve=False):
    torch.manual_seed(seed)
    m = KimiLinearSelfAttention(dim, H, max_seq_len=1024, head_dim=128, receives_ve=receives_ve)
    with torch.no_grad():
        for p in m.parameters():
            if p.dim() >= 2 and p.dtype == torch.bfloat16:
                p.copy_((torch.randn(p.shape) * (0.5 / p.shape[-1] ** 0.5)).bfloat16())
        m.dt_bias.copy_(torch.randn(m.dt_bias.shape) * 0.5)
        m.o_norm.weight.copy_((1 + 0.1 * torch.randn(m.o_norm.weight.shape)).bfloat16())
    return m.eval()


def _cpu_reference(m, x, ve=None):
    """The layer on the CPU: same PyTorch pieces, oracle gate + naive recurrence instead of the kernels."""
    B, T, _ = x.shape
    H, D = m.num_heads, m.head_k_dim
    q, _ = m.q_conv1d(m.q_proj(x))
    k, _ = m.k_conv1d(m.k_proj(x))
    v, _ = m.v_conv1d(m.v_proj(x))
    q, k, v = (t.view(B, T, H, D) for t in (q, k, v))
    if m.receives_ve:
        g_x = torch.sigmoid(m.g_ve).to(v.dtype)
        v = g_x * v + (1.0 - g_x) * ve.view_as(v)
    g = oracle.kda_gate(m.f_proj(x), m.A_log, D, m.dt_bias)
    beta = torch.sigmoid(m.b_proj(x)).float()
    o, _ = oracle.kda_recurrent(q, k, v, g.float(), beta, use_qk_l2norm=True)
    o = m.o_norm(o.to(torch.bfloat16), m.g_proj(x).view(B, T, H, D))
    return m.o_proj(o.reshape(B, T, H * D))


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
def test_short_convolution_kernel_matches_library_ops(B, T, C, K, bias, with_cache):
    """The streaming kernel against the same module on the CPU (grouped conv1d + SiLU in bf16)."""
    from daisy_amd.attention_kimi import ShortConvolution
    torch.manual_seed(T + C)
    m = ShortConvolution(C, K, bias=bias)
    if bias:
        with torch.no_grad():
            m.bias.copy_((torch.randn(C) * 0.3).bfloat16())
    x = torch.randn(B, T, C).bfloat16()
    cache = torch.randn(B, C, K).bfloat16() if with_cache else None
    with torch.no_grad():
        y_ref, c_ref = m(x, cache, output_final_state=True)
        md = ShortConvolution(C, K, bias=bias).to(DEV)
        md.load_state_dict(m.state_dict())
        y, c = md(x.to(DEV), None if cache is None else cache.to(DEV), output_final_state=True)
    assert y.shape == (B, T, C) and c.shape == (B, C, K)
    assert torch.equal(c.cpu(), c_ref), "carried window differs"
    # identical up to one bf16 rounding of the pre-activation (the summation order may differ)
    err = (y.float().cpu() - y_ref.float()).abs()
    tol = 2.0 ** -7 * y_ref.float().abs().clamp_min(0.25)
    say(f"short conv B{B} T{T} C{C} K{K}: max-abs {err.max().item():.3e}, mismatching {(err > 0).float().mean().item():.2%}")
    assert bool((err <= tol).all())
    # a sequence cut in two with the window carried equals the sequence in one go
    if T >= 2:
        with torch.no_grad():
            h = T // 2
            y1, c1 = md(x[:, :h].to(DEV), None if cache is None else cache.to(DEV), output_final_state=True)
            y2, c2 = md(x[:, h:].to(DEV), c1, output_final_state=True)
        assert torch.equal(torch.cat([y1, y2], dim=1), y) and torch.equal(c2, c)


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


@pytest.mark.parametrize("rows,D", [(5, 128), (1000, 128), (77, 64)])
def test_gated_rmsnorm_kernel_matches_formula(rows, D):
    from daisy_amd.attention_kimi import GatedRMSNorm
    torch.manual_seed(rows)
    m = GatedRMSNorm(D)
    with torch.no_grad():
        m.weight.copy_((1 + 0.2 * torch.randn(D)).bfloat16())
    x, g = torch.randn(rows, D).bfloat16() * 3, torch.randn(rows, D).bfloat16() * 2
    with torch.no_grad():
        ref = m(x, g)
        md = GatedRMSNorm(D).to(DEV)
        md.load_state_dict(m.state_dict())
        out = md(x.to(DEV), g.to(DEV))
    err = (out.float().cpu() - ref.float()).abs()
    say(f"gated norm rows{rows} D{D}: max-abs {err.max().item():.3e}")
    assert bool((err <= 2.0 ** -7 * ref.float().abs().clamp_min(1e-3)).all())
