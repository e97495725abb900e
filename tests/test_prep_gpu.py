"""Fused pre-attention pass (RMS norm + RoPE + ve mix) vs the oracle's bf16 chain, through the C ABI.

The oracle evaluates ``rms_norm -> apply_rope`` and ``g*v + (1-g)*ve`` on bf16 tensors, rounding
where the reference materialises a bf16 tensor; the kernel reproduces those roundings, so the two
agree bit for bit except where an fp32 intermediate sits on a bf16 rounding boundary (the
reciprocal square root of the GPU differs from the CPU's in the last fp32 bit).
"""
import pytest
import torch

import oracle
from daisy_amd import ops
from daisy_amd.functional import NORM_EPS_BF16
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _reference(q, k, v, cos, sin, pos0, ve, g_logit):
    T = q.shape[1]
    qn, kn, vn = oracle.rms_norm(q), oracle.rms_norm(k), oracle.rms_norm(v)
    if cos is not None:
        c, s = cos[pos0:pos0 + T], sin[pos0:pos0 + T]
        qn, kn = oracle.apply_rope(qn, c, s), oracle.apply_rope(kn, c, s)
    if ve is not None:
        vn = oracle.attention._mix_ve(vn, ve, g_logit)
    return qn, kn, vn


def _check(got, ref, what):
    g, r = got.float().cpu(), ref.float()
    assert_close_bf16(g, r, what, max_abs=4e-2, mean_abs=1e-4)     # one bf16 step at |x| <= 8 is 3.1e-2
    frac = (g != r).float().mean().item()
    assert frac <= 2e-3, f"{what}: {frac:.2e} of the elements differ from the bf16 chain"


@pytest.mark.parametrize("B,T,H,D,rope,mix,pos0", [
    (2, 37, 3, 128, True, True, 0),
    (1, 300, 4, 64, True, False, 0),
    (3, 1, 5, 128, True, True, 777),      # one decode step at position 777
    (2, 16, 2, 64, False, True, 0),
    (1, 5, 1, 128, False, False, 0),      # norm only, fewer rows than one workgroup
])
def test_prep_matches_bf16_chain(B, T, H, D, rope, mix, pos0):
    say(f"qkv_prep case B{B} T{T} H{H} D{D} rope={rope} mix={mix} pos0={pos0}")
    g = torch.Generator().manual_seed(B * 1000 + T)
    qkv = (torch.randn(B, T, 3 * H, D, generator=g) * 1.7).bfloat16()
    q, k, v = qkv.chunk(3, dim=-2)                      # strided views, as in the module
    ve = torch.randn(B, T, H, D, generator=g).bfloat16() if mix else None
    g_logit = 0.3228
    cos = sin = None
    if rope:
        cos, sin = oracle.rope_tables(D, pos0 + T + 3)
    q_ref, k_ref, v_ref = _reference(q, k, v, cos, sin, pos0, ve, g_logit if mix else None)

    qkv_d = qkv.to(DEV)
    qd, kd, vd = qkv_d.chunk(3, dim=-2)
    gate = torch.sigmoid(torch.tensor(g_logit)).bfloat16().float().reshape(1).to(DEV) if mix else None
    # k and v go straight into a [B, H, T, D] buffer (the layout prefill hands to the KV cache)
    k_bhtd = torch.full((B, H, T, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    v_bhtd = torch.full((B, H, T, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    q_out, k_out, v_out = ops.qkv_prep(qd, kd, vd, eps=NORM_EPS_BF16,
                                       cos=None if cos is None else cos.to(DEV), sin=None if sin is None else sin.to(DEV),
                                       pos0=pos0, ve=None if ve is None else ve.to(DEV), gate=gate,
                                       k_out=k_bhtd.transpose(1, 2), v_out=v_bhtd.transpose(1, 2))
    assert q_out.shape == (B, T, H, D) and q_out.is_contiguous()
    _check(q_out, q_ref, "q")
    _check(k_bhtd.transpose(1, 2), k_ref, "k")
    _check(v_bhtd.transpose(1, 2), v_ref, "v")
    assert torch.equal(qkv_d.cpu(), qkv), "inputs were modified"


def test_prep_matches_library_ops_on_gpu():
    """Same chain evaluated by the tensor library on the GPU (its own rms_norm kernel)."""
    B, T, H, D = 2, 257, 4, 128
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(B, T, 3 * H, D, generator=g).bfloat16().to(DEV)
    q, k, v = qkv.chunk(3, dim=-2)
    ve = torch.randn(B, T, H, D, generator=g).bfloat16().to(DEV)
    cos, sin = (t.to(DEV) for t in oracle.rope_tables(D, T))
    gl = torch.tensor(-1.5163, device=DEV)
    qn, kn, vn = (torch.nn.functional.rms_norm(t, (D,)) for t in (q, k, v))
    q_ref, k_ref = oracle.apply_rope(qn, cos, sin), oracle.apply_rope(kn, cos, sin)
    gx = torch.sigmoid(gl).to(torch.bfloat16)
    v_ref = gx * vn + (1.0 - gx) * ve
    q_out, k_out, v_out = ops.qkv_prep(q, k, v, eps=NORM_EPS_BF16, cos=cos, sin=sin, ve=ve, gate=gx.float().reshape(1))
    for got, ref, what in ((q_out, q_ref, "q"), (k_out, k_ref, "k"), (v_out, v_ref, "v")):
        _check(got, ref.cpu(), what)


def test_prep_at_device_position_equals_host_position():
    """Position read from device memory: same bits as the host-position entry point, for a decode
    row (T = 1) and a short run of rows, at several positions from one position tensor."""
    B, H, D, rows = 2, 3, 128, 300
    g = torch.Generator().manual_seed(11)
    cos, sin = (t.cuda() for t in oracle.rope_tables(D, rows))
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    for T in (1, 5):
        q, k, v, ve = (torch.randn(B, T, H, D, generator=g).bfloat16().cuda() for _ in range(4))
        gate = torch.sigmoid(torch.tensor(0.3)).bfloat16().float().reshape(1).cuda()
        for p0 in (0, 17, rows - T):
            say(f"prep_at case T{T} pos0 {p0}")
            pos.fill_(p0)
            want = ops.qkv_prep(q, k, v, eps=NORM_EPS_BF16, cos=cos, sin=sin, pos0=p0, ve=ve, gate=gate)
            got = ops.qkv_prep(q, k, v, eps=NORM_EPS_BF16, cos=cos, sin=sin, pos0=pos, ve=ve, gate=gate)
            for a, b, name in zip(got, want, "qkv"):
                assert torch.equal(a, b), f"{name} at pos0={p0}"
    with pytest.raises(ValueError):
        ops.qkv_prep(q, k, v, eps=NORM_EPS_BF16, pos0=pos)                      # no tables
    with pytest.raises(ValueError):
        ops.qkv_prep(q, k, v, eps=NORM_EPS_BF16, cos=cos, sin=sin, pos0=pos.long())


def test_prep_rejects_bad_arguments():
    q = torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops.qkv_prep(q, q, q, eps=1e-7, ve=q)                       # ve without gate
    with pytest.raises(TypeError):
        ops.qkv_prep(q.float(), q, q, eps=1e-7)
    q32 = torch.zeros(1, 4, 2, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="head_dim 32"):
        ops.qkv_prep(q32, q32, q32, eps=1e-7)
    cos = torch.zeros(3, 64, device=DEV)
    with pytest.raises(Exception, match="Rotary buffers too small"):
        ops.qkv_prep(q, q, q, eps=1e-7, cos=cos, sin=cos)
