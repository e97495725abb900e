"""Kernel 2 parity: HIP split-K decode vs the fp32 oracle (through the C ABI)."""
import pytest
import torch

import oracle
from daisy_amd import ops
from helpers import assert_close_bf16, say

pytestmark = pytest.mark.gpu


def _ref_decode(q, k_rows, v_rows, scale=0.12):
    """q [B,H,D]; rows [B,H,N,D] (already holding the new row) -> fp32 [B,H,D]."""
    return oracle.sdpa(q[:, :, None, :], k_rows, v_rows, None, scale)[:, :, 0, :]


@pytest.mark.parametrize("B,H,D,W,t,nsplit", [
    (2, 3, 128, 64, 10, 0),      # ring not yet wrapped
    (2, 3, 128, 64, 63, 0),      # last free slot
    (2, 3, 128, 64, 64, 0),      # first wrap: new row overwrites slot 0
    (1, 2, 128, 1024, 5000, 0),  # wrapped several times, auto split
    (1, 2, 128, 1024, 5000, 1),  # same, one workgroup per (b, h)
    (1, 2, 128, 1024, 5000, 4),
    (3, 2, 64, 200, 777, 0),     # D = 64, W not a multiple of the row block
    (3, 2, 64, 200, 777, 3),
    (1, 1, 128, 1, 9, 0),        # W = 1: only the new row
    (4, 8, 128, 4096, 8192, 0),  # the benchmark's ring shape at small batch
    (1, 12, 128, 8192, 8292, 0),   # one sequence, 12 heads, ring of 8192 (model_specs/daisy_milli.yml; the generator's batch of one)
    (1, 12, 128, 8192, 8292, 16),
    (1, 12, 128, 8192, 300, 0),    # the same ring early in a generation: 301 live rows
    (1, 12, 128, 8192, 8292, 64),  # the largest split count: every combine thread takes its full share of partials
    (1, 12, 128, 8192, 8292, 100), # more than that is taken as 64
    (1, 3, 64, 4096, 5000, 37),    # odd counts: combine groups with unequal numbers of splits
    (2, 2, 128, 2048, 3000, 9),
    (2, 2, 64, 2048, 3000, 5),     # fewer splits than combine groups at D = 64
])
def test_decode_ring_matches_oracle(B, H, D, W, t, nsplit):
    say(f"decode ring case B{B} H{H} D{D} W{W} t{t} nsplit{nsplit}")
    g = torch.Generator().manual_seed(W + t)
    kc = torch.randn(B, H, W, D, generator=g).bfloat16()
    vc = torch.randn(B, H, W, D, generator=g).bfloat16()
    q, kn, vn = (torch.randn(B, H, D, generator=g).bfloat16() for _ in range(3))
    cos, sin = oracle.rope_tables(D, t + 1)
    q_rot = oracle.apply_rope(q[:, None], cos[t:t + 1], sin[t:t + 1])[:, 0]
    k_rot = oracle.apply_rope(kn[:, None], cos[t:t + 1], sin[t:t + 1])[:, 0]
    n_rows, slot = min(t + 1, W), t % W
    k_exp, v_exp = kc.clone(), vc.clone()
    k_exp[:, :, slot] = k_rot
    v_exp[:, :, slot] = vn
    ref = _ref_decode(q_rot, k_exp[:, :, :n_rows], v_exp[:, :, :n_rows])

    dkc, dvc = kc.cuda(), vc.cuda()
    o = ops.decode_attention(q.cuda(), kn.cuda(), vn.cuda(), dkc, dvc, n_rows=n_rows, new_idx=slot,
                             write_back=True, cos_row=cos[t].cuda(), sin_row=sin[t].cuda(), nsplit=nsplit)
    torch.cuda.synchronize()
    assert_close_bf16(o, ref, "o")
    assert torch.equal(dkc.cpu(), k_exp), "cache K after the step (only the new slot may change)"
    assert torch.equal(dvc.cpu(), v_exp), "cache V after the step"


@pytest.mark.parametrize("n,window", [(0, 8), (5, 8), (20, 8), (20, None), (300, 257)])
def test_decode_chronological_context(n, window):
    """The reference's calling convention: k_ctx [B, n, H, D] + new row, last window-1 rows live."""
    B, H, D = 2, 2, 128
    say(f"decode ctx case n{n} window{window}")
    g = torch.Generator().manual_seed(n)
    k_ctx = torch.randn(B, n, H, D, generator=g).bfloat16()
    v_ctx = torch.randn(B, n, H, D, generator=g).bfloat16()
    q, kn, vn = (torch.randn(B, H, D, generator=g).bfloat16() for _ in range(3))
    r = n if window is None else min(n, max(window - 1, 0))
    k_all = torch.cat([k_ctx[:, n - r:], kn[:, None]], 1).transpose(1, 2)
    v_all = torch.cat([v_ctx[:, n - r:], vn[:, None]], 1).transpose(1, 2)
    ref = _ref_decode(q, k_all, v_all)
    dk, dv = k_ctx.cuda(), v_ctx.cuda()
    kc = dk[:, n - r:].transpose(1, 2) if r > 0 else None
    vc = dv[:, n - r:].transpose(1, 2) if r > 0 else None
    o = ops.decode_attention(q.cuda(), kn.cuda(), vn.cuda(), kc, vc, n_rows=r + 1, new_idx=r, write_back=False)
    assert_close_bf16(o, ref, "o")
    assert torch.equal(dk.cpu(), k_ctx) and torch.equal(dv.cpu(), v_ctx), "context must not be written"


def test_decode_consecutive_steps_append_in_place():
    """32 steps on one preallocated ring: every output checked, no host copies in between."""
    B, H, D, W, t0, steps = 2, 4, 128, 256, 500, 32
    g = torch.Generator().manual_seed(5)
    kc = torch.randn(B, H, W, D, generator=g).bfloat16()
    vc = torch.randn(B, H, W, D, generator=g).bfloat16()
    dkc, dvc = kc.cuda(), vc.cuda()
    ws = torch.empty(max(ops.decode_workspace_bytes(B, H, D, W), 1), dtype=torch.uint8, device="cuda:0")
    for s in range(steps):
        t = t0 + s
        q, kn, vn = (torch.randn(B, H, D, generator=g).bfloat16() for _ in range(3))
        slot = t % W
        kc[:, :, slot], vc[:, :, slot] = kn, vn
        ref = _ref_decode(q, kc, vc)
        o = ops.decode_attention(q.cuda(), kn.cuda(), vn.cuda(), dkc, dvc, n_rows=W, new_idx=slot,
                                 write_back=True, workspace=ws)
        assert_close_bf16(o, ref, f"o at step {s}")
    assert torch.equal(dkc.cpu(), kc) and torch.equal(dvc.cpu(), vc)


@pytest.mark.parametrize("B,H,D,W,nsplit", [(2, 3, 128, 64, 0), (1, 2, 128, 1024, 0), (1, 2, 128, 1024, 4), (3, 2, 64, 200, 3)])
def test_decode_at_device_position_matches_oracle(B, H, D, W, nsplit):
    """The position comes from device memory: one set of launch arguments serves an empty ring, a
    partly filled one (most splits empty), the last free slot and wrapped positions."""
    g = torch.Generator().manual_seed(W + D)
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    for t in (0, 1, 7, W // 2, W - 1, W, W + 1, 5 * W + 3):
        say(f"decode_at case B{B} H{H} D{D} W{W} nsplit{nsplit} t{t}")
        kc = torch.randn(B, H, W, D, generator=g).bfloat16()
        vc = torch.randn(B, H, W, D, generator=g).bfloat16()
        q, kn, vn = (torch.randn(B, H, D, generator=g).bfloat16() for _ in range(3))
        n_rows, slot = min(t + 1, W), t % W
        k_exp, v_exp = kc.clone(), vc.clone()
        k_exp[:, :, slot] = kn
        v_exp[:, :, slot] = vn
        ref = _ref_decode(q, k_exp[:, :, :n_rows], v_exp[:, :, :n_rows])
        dkc, dvc = kc.cuda(), vc.cuda()
        pos.fill_(t)
        o = ops.decode_attention_at(q.cuda(), kn.cuda(), vn.cuda(), dkc, dvc, pos, nsplit=nsplit)
        torch.cuda.synchronize()
        assert_close_bf16(o, ref, f"o at t={t}")
        assert torch.equal(dkc.cpu(), k_exp), "cache K after the step (only the new slot may change)"
        assert torch.equal(dvc.cpu(), v_exp), "cache V after the step"
        if n_rows == W:
            # full ring: same splits as the host-position entry point, so the same bits
            o_host = ops.decode_attention(q.cuda(), kn.cuda(), vn.cuda(), kc.cuda(), vc.cuda(), n_rows=W, new_idx=slot,
                                          write_back=True, nsplit=nsplit)
            assert torch.equal(o, o_host), "device- and host-position entry points differ on a full ring"


@pytest.mark.parametrize("ring_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,D,W,mix,nsplit", [(2, 3, 128, 64, True, 0), (1, 2, 128, 1024, False, 4), (3, 2, 64, 200, True, 3),
                                                (16, 8, 128, 4096, True, 0)])
def test_attn_step_prepares_rows_and_attends_in_one_launch(B, H, D, W, mix, nsplit, ring_dtype):
    """daisy_attn_step_fwd against the oracle's chain (norm, RoPE, value-embedding mix on bf16
    tensors, then fp32 attention over the ring with the new rows in slot t % W), with the position
    as a launch argument and in device memory; and against the two-kernel path.  The ring is bf16
    or fp16 (the reference generator's default cache dtype; bf16 rows convert to it without loss)."""
    from daisy_amd.functional import NORM_EPS_BF16
    g = torch.Generator().manual_seed(W + D + B)
    cos, sin = oracle.rope_tables(D, 6 * W + 8)
    g_logit = -0.4
    gate = torch.sigmoid(torch.tensor(g_logit)).bfloat16().float().reshape(1).cuda() if mix else None
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    for t in (0, 3, W - 1, W, 5 * W + 3):
        say(f"attn_step case B{B} H{H} D{D} W{W} mix{mix} nsplit{nsplit} t{t}")
        # (values below fp16's normal range would not survive the conversion of the random fill)
        kc, vc = (torch.randn(B, H, W, D, generator=g).bfloat16().to(ring_dtype).bfloat16() for _ in range(2))
        qkv = (torch.randn(B, 3 * H, D, generator=g) * 1.7).bfloat16()
        q, k, v = qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:]
        ve = torch.randn(B, H, D, generator=g).bfloat16() if mix else None
        qn = oracle.apply_rope(oracle.rms_norm(q)[:, None], cos[t:t + 1], sin[t:t + 1])[:, 0]
        kn = oracle.apply_rope(oracle.rms_norm(k)[:, None], cos[t:t + 1], sin[t:t + 1])[:, 0]
        vn = oracle.rms_norm(v)
        if mix:
            vn = oracle.attention._mix_ve(vn, ve, g_logit)
        n_rows, slot = min(t + 1, W), t % W
        k_exp, v_exp = kc.clone(), vc.clone()
        k_exp[:, :, slot], v_exp[:, :, slot] = kn, vn
        ref = _ref_decode(qn, k_exp[:, :, :n_rows], v_exp[:, :, :n_rows])
        qkv_d = qkv.cuda()
        rows = (qkv_d[:, :H], qkv_d[:, H:2 * H], qkv_d[:, 2 * H:])
        kw = dict(cos=cos.cuda(), sin=sin.cuda(), eps=NORM_EPS_BF16, ve=None if ve is None else ve.cuda(), gate=gate, nsplit=nsplit)
        outs = []
        for where in ("host", "device"):
            dk, dv = kc.cuda().to(ring_dtype), vc.cuda().to(ring_dtype)
            pos.fill_(t)
            o = ops.attn_step(*rows, dk, dv, t if where == "host" else pos, **kw)
            assert_close_bf16(o, ref, f"o, position on the {where}, t={t}")
            # the stored rows: the bf16 chain's, except where an fp32 sum sits on a rounding boundary
            for got, want, name in ((dk, k_exp, "K"), (dv, v_exp, "V")):
                assert got.dtype == ring_dtype
                got = got.float().cpu()
                want = want.float()
                assert torch.equal(got[:, :, :slot], want[:, :, :slot]) and torch.equal(got[:, :, slot + 1:], want[:, :, slot + 1:])
                row, row_ref = got[:, :, slot], want[:, :, slot]
                assert (row - row_ref).abs().max() <= 4e-2 and (row != row_ref).float().mean() <= 5e-3, f"new {name} row, t={t}"
            outs.append((o, dk, dv))
        assert torch.equal(outs[0][1], outs[1][1]) and torch.equal(outs[0][2], outs[1][2]), "host and device position store different rows"
        # the two-kernel path: same rows up to the order of the sums in the norm, same attention
        q2, k2, v2 = ops.qkv_prep(*(r.unsqueeze(1) for r in rows), eps=NORM_EPS_BF16, cos=kw["cos"], sin=kw["sin"], pos0=t,
                                  ve=None if ve is None else kw["ve"].unsqueeze(1), gate=gate)
        dk, dv = kc.cuda(), vc.cuda()
        o2 = ops.decode_attention(q2[:, 0], k2[:, 0], v2[:, 0], dk, dv, n_rows=n_rows, new_idx=slot, write_back=True, nsplit=nsplit)
        assert_close_bf16(outs[0][0], o2.float(), f"one launch vs two, t={t}", max_abs=8e-3, mean_abs=3e-4)


def test_decode_rejects_bad_arguments():
    z = torch.zeros(1, 1, 128, dtype=torch.bfloat16, device="cuda:0")
    rows = torch.zeros(1, 1, 4, 128, dtype=torch.bfloat16, device="cuda:0")
    with pytest.raises(RuntimeError, match="new_idx"):
        ops.decode_attention(z, z, z, rows, rows, n_rows=4, new_idx=4, write_back=False)
    with pytest.raises(RuntimeError, match="head_dim"):
        y = torch.zeros(1, 1, 33, dtype=torch.bfloat16, device="cuda:0")
        ops.decode_attention(y, y, y, None, None, n_rows=1, new_idx=0, write_back=False)


@pytest.mark.parametrize("D,n_rows,rope", [(8, 13, True), (2, 5, True), (32, 70, False), (200, 9, True)])
def test_decode_small_head_dims(D, n_rows, rope):
    """Head dims other than 64/128 (the reference's own unit tests use 2 and 8): the one-wavefront kernel."""
    B, H = 2, 3
    g = torch.Generator().manual_seed(D + n_rows)
    kc = torch.randn(B, H, n_rows, D, generator=g).bfloat16()
    vc = torch.randn(B, H, n_rows, D, generator=g).bfloat16()
    q, kn, vn = (torch.randn(B, H, D, generator=g).bfloat16() for _ in range(3))
    new_idx = n_rows // 2
    cos = sin = None
    qr, knr = q, kn
    if rope:
        cos_t, sin_t = oracle.rope_tables(D, 40)
        cos, sin = cos_t[17].contiguous(), sin_t[17].contiguous()
        qr = oracle.apply_rope(q[:, None], cos[None], sin[None])[:, 0]
        knr = oracle.apply_rope(kn[:, None], cos[None], sin[None])[:, 0]
    ke, ve = kc.clone(), vc.clone()
    ke[:, :, new_idx], ve[:, :, new_idx] = knr, vn
    ref = oracle.sdpa(qr[:, :, None], ke, ve, None, 0.12)[:, :, 0]
    dk, dv = kc.cuda(), vc.cuda()
    o = ops.decode_attention(q.cuda(), kn.cuda(), vn.cuda(), dk, dv, n_rows=n_rows, new_idx=new_idx, write_back=True,
                             cos_row=None if cos is None else cos.cuda(), sin_row=None if sin is None else sin.cuda())
    assert_close_bf16(o, ref, f"o (D={D})")
    assert torch.equal(dk.cpu(), ke) and torch.equal(dv.cpu(), ve), "the new row must be appended rotated, bit for bit"
