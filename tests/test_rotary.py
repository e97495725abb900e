"""RoPE tables of the drop-in module: the reference's formula and fp32 storage whatever the module is cast or moved
to (on the CPU, and under the ``gpu`` mark on ``cuda:0``, where the kernels read them)."""
import pytest
import torch

import oracle
from daisy_amd.attention import Rotary


DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("device", DEVICES)
def test_tables_follow_the_reference_formula(device):
    # models/daisy/attention.py:27-49: first D/4 frequencies (1/1024)**linspace(0,1,D/4), the rest zero
    for D in (64, 128, 8, 2):
        r = Rotary(D, 37).to(device)
        cos, sin = oracle.rope_tables(D, 37, base=1024.0, half_truncate=True)
        assert r.cos.device == torch.device(device)
        assert torch.equal(r.cos.cpu(), cos) and torch.equal(r.sin.cpu(), sin)
        assert r.cos.shape == (37, D // 2) and r.cos.dtype == torch.float32


@pytest.mark.parametrize("device", DEVICES)
def test_tables_stay_fp32_under_module_casts(device):
    r = Rotary(128, 50).to(device)
    cos0, sin0 = r.cos.clone(), r.sin.clone()
    for cast in (lambda m: m.bfloat16(), lambda m: m.half(), lambda m: m.to(torch.bfloat16), lambda m: m.float()):
        r = cast(r)
        assert r.cos.dtype == r.sin.dtype == r.inv_freq.dtype == torch.float32
        assert torch.equal(r.cos, cos0) and torch.equal(r.sin, sin0)
    assert "cos" not in r.state_dict() and "sin" not in r.state_dict()   # non-persistent, as in the reference
