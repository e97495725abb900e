"""Ring-buffer KV cache with the reference's interface (inference/kv_cache.py:4-68).

Storage is ``k, v [L, B, H, W, D]``; the token at absolute position ``p`` lives
in slot ``p % W``.  On top of the reference's methods the cache hands out a
``RingContext`` per layer so that the decode kernel can stream the ring in place
(physical order) and append the new row itself, instead of receiving a
chronological copy.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class RingContext:
    """Handle to one layer of a ``KVCache`` for the in-place decode path.

    ``k``/``v`` are the layer's ``[B, H, W, D]`` storage (views, not copies) and
    ``t`` the number of positions written so far; the row for position ``t``
    goes to slot ``t % W``.
    """
    cache: "KVCache"
    layer: int
    k: torch.Tensor
    v: torch.Tensor
    t: int
    W: int

    def mark_written(self) -> None:
        self.cache._staged[self.layer] = True


class KVCache:
    def __init__(self, L, B, H, W, D, device, dtype):
        self.H = H
        self.B = B
        self.D = D
        self.W = W
        self.L = L
        self.t = 0
        self.device = device
        self.dtype = dtype
        self.k = torch.zeros(L, B, H, W, D, device=device, dtype=dtype)
        self.v = torch.zeros(L, B, H, W, D, device=device, dtype=dtype)
        self._staged = [False] * L

    def reset_history(self):
        # The reference allocates fresh zero tensors here (kv_cache.py:19-23); the
        # storage is reused instead so that a long-lived cache never reallocates.
        self.k.zero_()
        self.v.zero_()
        self.t = 0
        self._staged = [False] * self.L

    def view(self, layer):
        """Chronological last ``min(t + staged, W)`` rows as ``[B, n, H, D]``."""
        staged = 1 if self._staged[layer] else 0
        m = self.t + staged
        n = min(m, self.W)
        if n == 0:
            return self.k[layer, :, :, :0, :].transpose(1, 2), self.v[layer, :, :, :0, :].transpose(1, 2)
        end = (self.t + staged) % self.W
        start = (end - n) % self.W
        if start < end:
            k = self.k[layer, :, :, start:end, :]
            v = self.v[layer, :, :, start:end, :]
        else:
            k = torch.cat([self.k[layer, :, :, start:, :], self.k[layer, :, :, :end, :]], dim=2)
            v = torch.cat([self.v[layer, :, :, start:, :], self.v[layer, :, :, :end, :]], dim=2)
        return k.transpose(1, 2), v.transpose(1, 2)

    def ring(self, layer) -> RingContext:
        """In-place handle for the decode kernel (no copy)."""
        return RingContext(self, layer, self.k[layer], self.v[layer], self.t, self.W)

    def write(self, layer, k_new, v_new):
        """Stages the row of position ``t``; accepts ``[B, 1, H, D]`` or ``[B, H, 1, D]``."""
        if k_new.size(1) == 1:
            k_new = k_new.transpose(1, 2)
            v_new = v_new.transpose(1, 2)
        i = self.t % self.W
        self.k[layer, :, :, i:i + 1, :] = k_new
        self.v[layer, :, :, i:i + 1, :] = v_new
        self._staged[layer] = True

    def advance(self):
        self.t += 1
        self._staged = [False] * self.L

    def bulk_write_packed(self, kv, pos):
        """Stores the last ``min(pos, W - 1)`` positions of ``kv [2, L, B, H, T, D]``."""
        r = min(pos, max(self.W - 1, 0))
        if r > 0:
            idx = torch.arange(pos - r, pos, device=self.k.device) % self.W
            self.k[:, :, :, idx, :] = kv[0][:, :, :, pos - r:pos, :].to(self.dtype)
            self.v[:, :, :, idx, :] = kv[1][:, :, :, pos - r:pos, :].to(self.dtype)
        self.t = pos
        self._staged = [False] * self.L

    def bulk_write_layer(self, layer, k, v, pos):
        """Per-layer form of ``bulk_write_packed`` for ``k, v [B, H, T, D]``; does not move ``t``."""
        r = min(pos, max(self.W - 1, 0))
        if r > 0:
            idx = torch.arange(pos - r, pos, device=self.k.device) % self.W
            self.k[layer][:, :, idx, :] = k[:, :, pos - r:pos, :].to(self.dtype)
            self.v[layer][:, :, idx, :] = v[:, :, pos - r:pos, :].to(self.dtype)
