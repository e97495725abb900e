"""daisy_attn_layer_step_fwd: a layer's decode step in one call equals its three parts one after the other
(QKV projection, one-launch attention step, output projection: models/daisy/attention.py:181-202), bit for bit --
it launches the same kernels on the same data -- and leaves the same rows in the ring.  The parts themselves are
checked against the oracle in test_linear_gpu.py and test_decode_gpu.py."""
import pytest
import torch

from daisy_amd import _lib, ops
from daisy_amd.functional import NORM_EPS_BF16
from helpers import say
import oracle

pytestmark = pytest.mark.gpu


def _setup(B, H, D, W, seed, ring_dtype):
    g = torch.Generator().manual_seed(seed)
    dim = H * D
    x = torch.randn(B, 1, dim, generator=g).bfloat16().cuda()
    w = (torch.randn(4, dim, dim, generator=g) * dim ** -0.5).bfloat16().cuda()
    kr = torch.randn(B, H, W, D, generator=g).to(ring_dtype).cuda()
    vr = torch.randn(B, H, W, D, generator=g).to(ring_dtype).cuda()
    ve = torch.randn(B, H, D, generator=g).bfloat16().cuda()
    gate = torch.tensor([0.4375], dtype=torch.float32, device="cuda")
    cos, sin = (t.cuda() for t in oracle.rope_tables(D, 4 * W + 8))
    return x, w, kr, vr, ve, gate, cos, sin


@pytest.mark.parametrize("B,H,D,W,t,mix,on_device,ring_dtype", [
    (1, 12, 128, 8192, 8292, False, False, torch.bfloat16),   # the generator's batch of one (model_specs/daisy_milli.yml)
    (1, 12, 128, 8192, 300, True, True, torch.bfloat16),
    (3, 4, 64, 200, 777, True, False, torch.float16),
    (4, 2, 128, 64, 63, False, True, torch.bfloat16),
    (8, 2, 64, 32, 5, True, False, torch.bfloat16),            # the most rows the call takes
])
def test_layer_step_equals_its_three_parts(B, H, D, W, t, mix, on_device, ring_dtype):
    say(f"layer step B{B} H{H} D{D} W{W} t{t} mix{mix} device position {on_device} {ring_dtype}")
    x, w, kr, vr, ve, gate, cos, sin = _setup(B, H, D, W, seed=B * 100 + H, ring_dtype=ring_dtype)
    w_qkv, w_out = w[:3].flatten(end_dim=1), w[3]
    pos = torch.tensor([t], dtype=torch.int32, device="cuda") if on_device else t
    kw = dict(cos=cos, sin=sin, eps=NORM_EPS_BF16, ve=ve if mix else None, gate=gate if mix else None, scale=0.12)
    k1, v1 = kr.clone(), vr.clone()
    qkv = ops.linear_rows(x, w_qkv).view(B, 3 * H, D)
    o = ops.attn_step(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], k1, v1, pos, **kw)
    y_parts = ops.linear_rows(o.reshape(B, 1, H * D), w_out)
    k2, v2 = kr.clone(), vr.clone()
    y = ops.attn_layer_step(x, w_qkv, w_out, k2, v2, pos, **kw)
    assert y.shape == x.shape and torch.equal(y, y_parts)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    assert not torch.equal(k2[:, :, t % W], kr[:, :, t % W])      # the new row went into its slot


def test_layer_step_refusals():
    x, w, kr, vr, ve, gate, cos, sin = _setup(9, 2, 64, 16, seed=1, ring_dtype=torch.bfloat16)
    w_qkv, w_out = w[:3].flatten(end_dim=1), w[3]
    kw = dict(cos=cos, sin=sin, eps=NORM_EPS_BF16)
    with pytest.raises(RuntimeError, match="at most 8"):
        ops.attn_layer_step(x, w_qkv, w_out, kr, vr, 3, **kw)
    with pytest.raises(ValueError, match="do not fit"):
        ops.attn_layer_step(x[:2], w_qkv[:, :64], w_out, kr[:2], vr[:2], 3, **kw)
    with pytest.raises(TypeError):
        ops.attn_layer_step(x[:2].float(), w_qkv, w_out, kr[:2], vr[:2], 3, **kw)
    lib = _lib.load()
    need = lib.daisy_attn_layer_step_workspace_bytes(2, 2, 64, 16, 0)
    assert need >= 2 * 3 * 2 * 64 * 2 + 2 * 2 * 64 * 2 and need % 256 == 0
    small = torch.empty(256, dtype=torch.uint8, device="cuda")
    rc = lib.daisy_attn_layer_step_fwd(
        x.data_ptr(), 128, w_qkv.data_ptr(), 128, w_out.data_ptr(), 128, None, None, None, cos.data_ptr(), sin.data_ptr(),
        int(cos.shape[0]), 3, None, None, 1e-6, kr.data_ptr(), _lib.strides(kr, (0, 1, 2)), vr.data_ptr(),
        _lib.strides(vr, (0, 1, 2)), 0, x.data_ptr(), 128, 2, 2, 64, 128, 16, 0.12, 0, small.data_ptr(), 256, None)
    assert rc != 0 and "workspace" in lib.daisy_last_error().decode()
