"""The five benchmark configurations at their full sizes, on seeded inputs (torch.manual_seed(0) style generators).

Config 1 (the small fp32 plumbing layer) is test_module_gpu.py::test_config1_plumbing_layer.  The others are too
large for a full CPU evaluation, so the CPU oracle is evaluated on sampled query rows / (batch, head) pairs, and
the tensor library's fp32 ops on the GPU serve as a second, full-size check where that is cheap.
Tolerances: bf16 outputs max-abs <= 2e-2, mean-abs <= 2e-3; KDA final state relative error <= 1e-3.
"""
import pytest
import torch
import torch.nn.functional as F

import oracle
from daisy_amd import chunk_kda, ops
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SCALE = 0.12


def _rope_base10000(D, T):
    freq = (1.0 / 10000.0) ** torch.linspace(0, 1, steps=D // 2, dtype=torch.float32)
    theta = torch.arange(T, dtype=torch.float32)[:, None] * freq[None, :]
    return theta.cos(), theta.sin()


def _library_windowed_attention(q, k, v, window, scale, rows_per_block=1024):
    """EVERY row of windowed causal attention from the tensor library's fp32 ops on the GPU (matmul, softmax,
    matmul over the keys a block of queries can see): the full-size second check next to the CPU oracle's
    sampled rows.  q, k, v: [B, T, H, D] on the GPU; returns fp32 [B, T, H, D]."""
    B, T, H, D = q.shape
    W = T if window is None else window
    out = torch.empty(B, T, H, D, dtype=torch.float32, device=q.device)
    for b in range(B):
        qf, kf, vf = (t[b].transpose(0, 1).float() for t in (q, k, v))            # [H, T, D]
        for r0 in range(0, T, rows_per_block):
            r1 = min(r0 + rows_per_block, T)
            lo = max(0, r0 - W + 1)
            s_ = torch.matmul(qf[:, r0:r1], kf[:, lo:r1].transpose(1, 2)) * scale   # [H, rows, keys]
            d = torch.arange(r0, r1, device=q.device)[:, None] - torch.arange(lo, r1, device=q.device)[None, :]
            s_.masked_fill_(((d < 0) | (d >= W))[None], float("-inf"))
            out[b, r0:r1] = torch.matmul(torch.softmax(s_, dim=-1), vf[:, lo:r1]).transpose(0, 1)
    return out


def test_config2_windowed_prefill_full_size():
    """B8 T4096 d1024 H8 D128 W1024: merged QKV, q/k/v RMS-normed, RoPE base 10000, bf16."""
    B, T, H, D, W, dim = 8, 4096, 8, 128, 1024, 1024
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, T, dim, generator=g).bfloat16()
    w = (torch.randn(3 * dim, dim, generator=g) * 0.02).bfloat16()
    qkv = F.linear(x.to(DEV), w.to(DEV)).view(B, T, 3 * H, D)
    q, k, v = (F.rms_norm(t, (D,)) for t in qkv.chunk(3, dim=-2))
    cos, sin = _rope_base10000(D, T)
    o, k_rot = ops.prefill_attention(q, k, v, window=W, scale=SCALE, cos=cos.to(DEV), sin=sin.to(DEV))
    torch.cuda.synchronize()
    # rows around the start, the first full window, block and tile boundaries, and the end
    rows = torch.cat([torch.arange(0, 40), torch.arange(1000, 1050), torch.arange(2040, 2056), torch.arange(3071, 3090),
                      torch.arange(T - 40, T)])
    qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
    qr, kr = oracle.apply_rope(qc, cos, sin), oracle.apply_rope(kc, cos, sin)
    assert torch.equal(k_rot.cpu(), kr), "rotated keys differ from the elementwise expression"
    ref = oracle.windowed_attention_blockwise(qr.transpose(1, 2), kr.transpose(1, 2), vc.transpose(1, 2), W, SCALE, None, rows=rows)
    mx, mn = assert_close_bf16(o[:, rows.to(DEV)], ref.transpose(1, 2), "config 2 o[rows]")
    say(f"config 2: max-abs {mx:.2e} mean-abs {mn:.2e} over {rows.numel()} rows x {B * H} (batch, head)")
    # the one-pass norm + RoPE kernel followed by attention without tables gives the same result
    qp, kp, vp = ops.qkv_prep(*qkv.chunk(3, dim=-2), eps=torch.finfo(torch.float32).eps, cos=cos.to(DEV), sin=sin.to(DEV))
    o2, _ = ops.prefill_attention(qp, kp, vp, window=W, scale=SCALE)
    assert_close_bf16(o2[:, rows.to(DEV)], ref.transpose(1, 2), "config 2 (prep kernel) o[rows]")
    # every row of every (batch, head) against the library's fp32 ops on the GPU, itself checked against the
    # CPU oracle on the sampled rows
    lib = _library_windowed_attention(oracle.apply_rope(q, cos.to(DEV), sin.to(DEV)), k_rot, v, W, SCALE)
    assert (lib[:, rows.to(DEV)].cpu() - ref.transpose(1, 2)).abs().max().item() <= 1e-4
    mx, mn = assert_close_bf16(o, lib, "config 2 o, all rows")
    say(f"config 2, all {B * T * H} rows against fp32 library ops: max-abs {mx:.2e} mean-abs {mn:.2e}")


@pytest.mark.parametrize("window", [2048, None])
def test_config3_long_context_prefill_full_size(window):
    """B1 T65536 H16 D128, q/k/v ~ N(0,1) already rotated; window 2048 and full causal."""
    B, T, H, D = 1, 65536, 16, 128
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, T, H, D, generator=g).bfloat16() for _ in range(3))
    o, _ = ops.prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), window=window, scale=SCALE)
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, 8), torch.arange(2044, 2052), torch.arange(30000, 30008), torch.arange(46336, 46344),
                      torch.arange(T - 8, T)])
    ref = oracle.windowed_attention_blockwise(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), window, SCALE, None, rows=rows)
    mx, mn = assert_close_bf16(o[:, rows.to(DEV)], ref.transpose(1, 2), f"config 3 window={window} o[rows]")
    say(f"config 3 window={window}: max-abs {mx:.2e} mean-abs {mn:.2e}")
    assert torch.isfinite(o.float()).all()
    if window is not None:
        # every row against the library's fp32 ops on the GPU (a block of queries sees at most 2 * window keys)
        lib = _library_windowed_attention(q.to(DEV), k.to(DEV), v.to(DEV), window, SCALE, rows_per_block=2048)
        assert (lib[:, rows.to(DEV)].cpu() - ref.transpose(1, 2)).abs().max().item() <= 1e-4
        mx, mn = assert_close_bf16(o, lib, "config 3 window o, all rows")
        say(f"config 3 window={window}, all {T * H} rows against fp32 library ops: max-abs {mx:.2e} mean-abs {mn:.2e}")
    else:
        # full causal: every 64th row (offset 37, so tile and block edges rotate through) against the same ops
        sub = torch.arange(37, T, 64, device=DEV)
        qf, kf, vf = (t.to(DEV)[0].transpose(0, 1).float() for t in (q, k, v))
        for h0 in range(0, H, 4):
            s_ = torch.matmul(qf[h0:h0 + 4][:, sub], kf[h0:h0 + 4].transpose(1, 2)) * SCALE
            s_.masked_fill_((torch.arange(T, device=DEV)[None, :] > sub[:, None])[None], float("-inf"))
            lib = torch.matmul(torch.softmax(s_, dim=-1), vf[h0:h0 + 4]).transpose(0, 1)        # [rows, 4, D]
            assert_close_bf16(o[0, sub, h0:h0 + 4], lib, f"config 3 full causal, heads {h0}..{h0 + 3}, every 64th row")


def test_config4_decode_full_size_256_steps():
    """B64 H16 D128 ring of 4096 slots holding positions up to 8192; 256 consecutive steps, every step checked
    on sampled (batch, head) pairs against the CPU oracle and, at three steps, on every pair against fp32 library ops."""
    B, H, D, W, t0, steps = 64, 16, 128, 4096, 8192, 256
    gd = torch.Generator(device=DEV).manual_seed(0)
    kc = torch.randn(B, H, W, D, generator=gd, device=DEV).bfloat16()
    vc = torch.randn(B, H, W, D, generator=gd, device=DEV).bfloat16()
    pairs = [(0, 0), (17, 5), (63, 15), (31, 8)]
    bi = torch.tensor([p[0] for p in pairs])
    hi = torch.tensor([p[1] for p in pairs])
    k_cpu, v_cpu = kc[bi.to(DEV), hi.to(DEV)].cpu(), vc[bi.to(DEV), hi.to(DEV)].cpu()      # [P, W, D]
    ws = torch.empty(max(ops.decode_workspace_bytes(B, H, D, W), 1), dtype=torch.uint8, device=DEV)
    o = torch.empty(B, H, D, dtype=torch.bfloat16, device=DEV)
    worst = 0.0
    for s in range(steps):
        t = t0 + s
        slot = t % W
        q, kn, vn = (torch.randn(B, H, D, generator=gd, device=DEV).bfloat16() for _ in range(3))
        ops.decode_attention(q, kn, vn, kc, vc, n_rows=W, new_idx=slot, write_back=True, scale=SCALE, out=o, workspace=ws)
        k_cpu[:, slot], v_cpu[:, slot] = kn[bi.to(DEV), hi.to(DEV)].cpu(), vn[bi.to(DEV), hi.to(DEV)].cpu()
        ref = oracle.sdpa(q[bi.to(DEV), hi.to(DEV)].cpu()[:, None, None, :], k_cpu[:, None], v_cpu[:, None], None, SCALE)[:, 0, 0]
        mx, _ = assert_close_bf16(o[bi.to(DEV), hi.to(DEV)], ref, f"config 4 step {s}")
        worst = max(worst, mx)
        if s in (0, 127, 255):
            att = torch.softmax(torch.einsum("bhd,bhwd->bhw", q.float(), kc.float()) * SCALE, dim=-1)
            full = torch.einsum("bhw,bhwd->bhd", att, vc.float())
            assert_close_bf16(o, full.cpu(), f"config 4 step {s}, all (batch, head) pairs")
    say(f"config 4: worst max-abs over 256 steps {worst:.2e}")
    assert torch.equal(kc[bi.to(DEV), hi.to(DEV)].cpu(), k_cpu) and torch.equal(vc[bi.to(DEV), hi.to(DEV)].cpu(), v_cpu)


@pytest.mark.parametrize("ring_dtype", [torch.bfloat16, torch.float16])
def test_config4_decode_steps_in_one_launch(ring_dtype):
    """The configuration-4 ring (B64 H16 D128, 4096 slots, positions from 8192) through the one-launch step:
    rows straight from a QKV projection, norm + RoPE + append + attention in the kernel, position in
    device memory and counted up on the device, ring in bf16 and in the reference generator's fp16.
    32 consecutive steps, each checked on sampled (batch, head) pairs against the CPU oracle's chain."""
    from daisy_amd.functional import NORM_EPS_BF16
    B, H, D, W, t0, steps = 64, 16, 128, 4096, 8192, 32
    gd = torch.Generator(device=DEV).manual_seed(1)
    kc = torch.randn(B, H, W, D, generator=gd, device=DEV).bfloat16().to(ring_dtype)
    vc = torch.randn(B, H, W, D, generator=gd, device=DEV).bfloat16().to(ring_dtype)
    pairs = [(0, 0), (17, 5), (63, 15), (31, 8)]
    bi = torch.tensor([p[0] for p in pairs]).to(DEV)
    hi = torch.tensor([p[1] for p in pairs]).to(DEV)
    k_cpu, v_cpu = kc[bi, hi].float().cpu(), vc[bi, hi].float().cpu()      # [P, W, D]
    cos, sin = oracle.rope_tables(D, t0 + steps)
    cos_d, sin_d = cos.to(DEV), sin.to(DEV)
    pos = torch.full((1,), t0, dtype=torch.int32, device=DEV)
    ws = torch.empty(max(ops.decode_workspace_bytes(B, H, D, W), 1), dtype=torch.uint8, device=DEV)
    o = torch.empty(B, H, D, dtype=torch.bfloat16, device=DEV)
    worst = 0.0
    for s in range(steps):
        t = t0 + s
        slot = t % W
        qkv = (torch.randn(B, 3 * H, D, generator=gd, device=DEV) * 1.3).bfloat16()
        ops.attn_step(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], kc, vc, pos, cos=cos_d, sin=sin_d, eps=NORM_EPS_BF16,
                      scale=SCALE, out=o, workspace=ws)
        pos.add_(1)
        rows = [oracle.rms_norm(qkv[:, i * H:(i + 1) * H][bi, hi].cpu()) for i in range(3)]          # [P, D] each
        q_ref = oracle.apply_rope(rows[0][:, None, None], cos[t:t + 1], sin[t:t + 1])[:, 0, 0]
        k_ref = oracle.apply_rope(rows[1][:, None, None], cos[t:t + 1], sin[t:t + 1])[:, 0, 0]
        k_cpu[:, slot], v_cpu[:, slot] = k_ref.float(), rows[2].float()
        ref = oracle.sdpa(q_ref[:, None, None, :], k_cpu[:, None], v_cpu[:, None], None, SCALE)[:, 0, 0]
        mx, _ = assert_close_bf16(o[bi, hi], ref, f"config 4 one-launch step {s} ({ring_dtype})")
        worst = max(worst, mx)
    say(f"config 4, one launch per step, {ring_dtype}: worst max-abs over {steps} steps {worst:.2e}")
    assert int(pos) == t0 + steps and kc.dtype == ring_dtype
    got_k, got_v = kc[bi, hi].float().cpu(), vc[bi, hi].float().cpu()
    assert (got_k != k_cpu).float().mean() <= 1e-4 and (got_k - k_cpu).abs().max() <= 4e-2, "ring keys"
    assert (got_v != v_cpu).float().mean() <= 1e-4 and (got_v - v_cpu).abs().max() <= 4e-2, "ring values"


def test_config5_kda_full_size():
    """B4 T8192 H16 Dk=Dv=128 chunk 64: q, k L2-normalised, g = logsigmoid(N(0,1)), beta = sigmoid(N(0,1)), S0 = 0."""
    B, T, H, Dk = 4, 8192, 16, 128
    gd = torch.Generator(device=DEV).manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=gd, device=DEV)
    q = F.normalize(rn(B, T, H, Dk), dim=-1).bfloat16()
    k = F.normalize(rn(B, T, H, Dk), dim=-1).bfloat16()
    v = rn(B, T, H, Dk).bfloat16()
    gl = F.logsigmoid(rn(B, T, H, Dk))
    beta = torch.sigmoid(rn(B, T, H))
    o, S = chunk_kda(q, k, v, gl, beta, scale=Dk ** -0.5, output_final_state=True, use_qk_l2norm_in_kernel=True)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(S).all()
    for b, h in ((0, 0), (3, 15), (2, 7)):
        sl = lambda t: t[b:b + 1, :, h:h + 1].cpu()
        o_ref, S_ref = oracle.kda_recurrent(sl(q), sl(k), sl(v), sl(gl), beta[b:b + 1, :, h:h + 1].cpu())
        mx, mn = assert_close_bf16(o[b:b + 1, :, h:h + 1], o_ref, f"config 5 o (b={b}, h={h})")
        rel = ((S[b, h].cpu() - S_ref[0, 0]).norm() / S_ref[0, 0].norm()).item()
        say(f"config 5 (b={b}, h={h}): o max-abs {mx:.2e} mean-abs {mn:.2e}, state rel err {rel:.2e}")
        assert rel <= 1e-3
    _check_every_pair(q, k, v, gl, beta, o, S, "config 5")


def _check_every_pair(q, k, v, gl, beta, o, S, what):
    """Every (batch, head) pair, every token: the naive recurrence evaluated in fp32 on the same device tensors
    (the oracle's loop, library fp32 einsums) against the kernel's outputs and final states."""
    o_ref, S_ref = oracle.kda_recurrent(q, k, v, gl, beta)
    err = (o.float() - o_ref).abs()
    per_pair_max = err.amax(dim=(1, 3))                              # [B, H]
    per_pair_mean = err.mean(dim=(1, 3))
    rel = (S - S_ref).flatten(2).norm(dim=-1) / S_ref.flatten(2).norm(dim=-1)
    say(f"{what}, all {rel.numel()} (batch, head) pairs: o max-abs {per_pair_max.max().item():.2e}, worst mean-abs "
        f"{per_pair_mean.max().item():.2e}, worst state rel err {rel.max().item():.2e}")
    assert per_pair_max.max().item() <= 2e-2 and per_pair_mean.max().item() <= 2e-3
    assert rel.max().item() <= 1e-3


def test_config5_kda_full_size_with_the_layer_gate():
    """The configuration-5 shape with log-decays from the layer's own gate at its initial parameters
    (A_log = log U(1, 16), dt_bias = 0, models/daisy/attention_kimi.py:95-99,132): decays of e^-1 .. e^-20 per token,
    the steep path of the chunk kernel.  Every (batch, head) pair and token against the recurrence."""
    B, T, H, Dk = 4, 8192, 16, 128
    gd = torch.Generator(device=DEV).manual_seed(5)
    rn = lambda *s: torch.randn(*s, generator=gd, device=DEV)
    q = F.normalize(rn(B, T, H, Dk), dim=-1).bfloat16()
    k = F.normalize(rn(B, T, H, Dk), dim=-1).bfloat16()
    v = rn(B, T, H, Dk).bfloat16()
    A_log = torch.log(torch.empty(H, device=DEV).uniform_(1, 16, generator=gd))
    gl = oracle.kda_gate(rn(B, T, H * Dk), A_log, Dk)               # fp32 [B, T, H, Dk]
    beta = torch.sigmoid(rn(B, T, H))
    o, S = chunk_kda(q, k, v, gl, beta, scale=Dk ** -0.5, output_final_state=True, use_qk_l2norm_in_kernel=True)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(S).all()
    say(f"gate log-decays: mean {gl.mean().item():.2f}, min {gl.min().item():.1f}")
    _check_every_pair(q, k, v, gl, beta, o, S, "config 5 shape, layer gate")
