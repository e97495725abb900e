"""Elementwise helpers that stay in PyTorch (library routines on either side)."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor


def norm(x: Tensor) -> Tensor:
    """Weightless RMS norm over the last dim with the library's default eps.

    Same call as the reference's ``norm`` (models/daisy/functional.py:6-7): no eps is passed, and torch 2.10
    then adds the machine epsilon of its accumulation type -- fp32's for bf16 and fp32 inputs alike, on the
    CPU and on the GPU -- not ``finfo(x.dtype).eps`` (see ``NORM_EPS_BF16`` below).
    """
    return F.rms_norm(x, (x.size(-1),))


# What ``F.rms_norm(x, (D,))`` adds to mean(x^2) when no eps is passed: the machine epsilon of
# the accumulation type, which is fp32 for bf16 inputs (torch 2.10).  The fused pre-attention
# kernel takes the same value so that it rounds like ``norm``.
NORM_EPS_BF16 = torch.finfo(torch.float32).eps


@torch.no_grad()
def init_linear(w: Tensor) -> Tensor:
    """Uniform init with std 0.5 / sqrt(fan_in) (models/daisy/functional.py:10-14)."""
    bound = (3 ** 0.5) * 0.5 * (w.size(-1) ** -0.5)
    return w.uniform_(-bound, bound)
