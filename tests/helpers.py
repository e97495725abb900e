"""Shared helpers for the parity tests."""
from __future__ import annotations

import torch

# Tolerances for bf16 kernels against the fp32 oracle (max-abs, mean-abs).
BF16_MAX_ABS = 2e-2
BF16_MEAN_ABS = 2e-3


def assert_close_bf16(got: torch.Tensor, ref: torch.Tensor, what: str = "",
                      max_abs: float = BF16_MAX_ABS, mean_abs: float = BF16_MEAN_ABS):
    g = got.detach().float().cpu()
    r = ref.detach().float().cpu()
    assert g.shape == r.shape, f"{what}: shape {tuple(g.shape)} vs {tuple(r.shape)}"
    assert torch.isfinite(g).all(), f"{what}: non-finite values in kernel output"
    err = (g - r).abs()
    mx, mn = err.max().item(), err.mean().item()
    assert mx <= max_abs and mn <= mean_abs, f"{what}: max-abs {mx:.3e} (<= {max_abs}), mean-abs {mn:.3e} (<= {mean_abs})"
    return mx, mn


def say(msg: str):
    print(msg, flush=True)
