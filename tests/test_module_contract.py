"""Constructor contract of the drop-in ``CausalSelfAttention`` (models/daisy/attention.py:73-110): parameter names,
shapes, dtypes and initial values are what a checkpoint of the reference and its optimizer groups rely on.  Runs on
the CPU and, under the ``gpu`` mark, on a module moved to ``cuda:0``."""
import pytest
import torch

from daisy_amd import CausalSelfAttention

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("receives_ve", [False, True])
def test_state_dict_keys_shapes_and_dtypes(device, receives_ve, monkeypatch):
    monkeypatch.delenv("DISABLE_O_ZERO_INIT", raising=False)
    dim, H, D = 256, 4, 64
    attn = CausalSelfAttention(dim=dim, num_heads=H, head_dim=D, receives_ve=receives_ve, layer_idx=0, max_seq_len=64).to(device)
    sd = attn.state_dict()
    # attention.py:82 (qkvo_w), :104/:106 (g_ve); the rotary tables are non-persistent buffers (attention.py:45-47)
    assert set(sd.keys()) == ({"qkvo_w", "g_ve"} if receives_ve else {"qkvo_w"})
    assert set(n for n, _ in attn.named_parameters()) == set(sd.keys())
    w = sd["qkvo_w"]
    assert tuple(w.shape) == (4, dim, dim) and w.dtype == torch.bfloat16 and w.device == torch.device(device)
    assert float(w[3].float().abs().sum()) == 0.0                        # attention.py:83-84: the output projection starts at zero
    bound = (3 ** 0.5) * 0.5 * dim ** -0.5                              # functional.py:11-14
    q = w[:3].float()
    assert float(q.abs().max()) <= bound * 1.01
    assert abs(float(q.std()) - 0.5 * dim ** -0.5) <= 0.02 * 0.5 * dim ** -0.5
    if receives_ve:
        assert sd["g_ve"].shape == () and sd["g_ve"].dtype == torch.float32
        assert abs(float(sd["g_ve"]) - 0.3228) < 1e-6                    # layer 0's gate logit, attention.py:95
    assert attn.attn_scale == 0.12 and attn.num_heads == H and attn.head_dim == D and attn.m_dim == dim
    assert attn.rotary.cos.dtype == torch.float32 and attn.rotary.cos.device == torch.device(device)


@pytest.mark.parametrize("device", DEVICES)
def test_gate_logits_per_layer_and_the_unit_test_switch(device, monkeypatch):
    want = {0: 0.3228, 1: 0.0, 2: -1.5163, 21: -2.4423, 22: -2.9444, 23: 10.0, 7: 0.0, None: 0.0}
    for layer, val in want.items():
        attn = CausalSelfAttention(128, 2, 64, receives_ve=True, layer_idx=layer, max_seq_len=16).to(device)
        assert abs(float(attn.g_ve.detach()) - val) < 1e-6
    assert CausalSelfAttention(128, 2, 64, receives_ve=False, max_seq_len=16).g_ve is None
    monkeypatch.setenv("DISABLE_O_ZERO_INIT", "1")                      # attention.py:83: the reference's unit tests keep W[3]
    attn = CausalSelfAttention(128, 2, 64, max_seq_len=16).to(device)
    assert float(attn.qkvo_w[3].float().abs().sum()) > 0.0


@pytest.mark.parametrize("device", DEVICES)
def test_a_reference_state_dict_loads(device):
    """A state dict with the reference's keys and shapes loads strictly, onto either device."""
    dim = 128
    src = {"qkvo_w": torch.randn(4, dim, dim).bfloat16(), "g_ve": torch.tensor(0.25)}
    attn = CausalSelfAttention(dim, 2, 64, receives_ve=True, max_seq_len=16).to(device)
    missing, unexpected = attn.load_state_dict(src, strict=True)
    assert not missing and not unexpected
    assert torch.equal(attn.qkvo_w.detach().cpu(), src["qkvo_w"]) and float(attn.g_ve.detach()) == 0.25
    with pytest.raises((RuntimeError, AssertionError)):
        CausalSelfAttention(dim, 3, 64, max_seq_len=16)                 # attention.py:76: dim % num_heads


def test_kimi_layer_constructor_contract():
    """KimiLinearSelfAttention (models/daisy/attention_kimi.py:64-110): the reference's parameter names, shapes and
    dtypes at head widths other than 128, and a clear refusal of what the kernels under the layer do not serve."""
    from daisy_amd import KimiLinearSelfAttention
    m = KimiLinearSelfAttention(256, 4, max_seq_len=64, head_dim=64, expand_v=2.0, conv_size=3)
    assert (m.head_k_dim, m.head_v_dim, m.key_dim, m.value_dim) == (64, 128, 256, 512)      # attention_kimi.py:79-82
    sd = m.state_dict()
    assert sd["q_proj.weight"].shape == (256, 256) and sd["v_proj.weight"].shape == (512, 256)
    assert sd["q_conv1d.weight"].shape == (256, 1, 3) and sd["v_conv1d.weight"].shape == (512, 1, 3)
    assert sd["f_proj.0.weight"].shape == (128, 256) and sd["f_proj.1.weight"].shape == (256, 128)
    assert sd["g_proj.1.weight"].shape == (512, 128) and sd["g_proj.1.bias"].shape == (512,)
    assert sd["o_norm.weight"].shape == (128,) and sd["o_proj.weight"].shape == (256, 512)
    assert sd["A_log"].shape == (1, 1, 4, 1) and sd["A_log"].dtype == torch.float32 and sd["dt_bias"].shape == (256,)
    assert sd["b_proj.weight"].shape == (4, 256) and sd["q_proj.weight"].dtype == torch.bfloat16
    for kw in (dict(head_dim=160), dict(head_dim=36), dict(head_dim=128, expand_v=0.75), dict(head_dim=128, conv_size=5)):
        with pytest.raises(ValueError, match="not supported"):
            KimiLinearSelfAttention(256, 2, max_seq_len=64, **kw)
