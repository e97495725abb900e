"""Ring-buffer KV cache semantics restated with plain Python indexing.

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

Follows inference/kv_cache.py:4-68.  Storage is a numpy array
``[L, B, H, W, D]`` per tensor and every operation is written as an explicit
loop over absolute positions so that the slot arithmetic (``p % W``) is in one
obvious place.
"""
from __future__ import annotations

import numpy as np


class RingKVCache:
    def __init__(self, L: int, B: int, H: int, W: int, D: int, dtype=np.float32):
        self.L, self.B, self.H, self.W, self.D = L, B, H, W, D
        self.dtype = dtype
        self.reset_history()

    def reset_history(self):
        # inference/kv_cache.py:19-23
        shape = (self.L, self.B, self.H, self.W, self.D)
        self.k = np.zeros(shape, dtype=self.dtype)
        self.v = np.zeros(shape, dtype=self.dtype)
        self.t = 0
        self.staged = [False] * self.L

    def view(self, layer: int):
        """Chronological last ``min(t + staged, W)`` rows as ``[B, n, H, D]``.

        inference/kv_cache.py:26-42: the newest visible absolute position is
        ``t - 1`` (or ``t`` when a write for this step is staged).
        """
        m = self.t + (1 if self.staged[layer] else 0)
        n = min(m, self.W)
        k = np.zeros((self.B, n, self.H, self.D), dtype=self.dtype)
        v = np.zeros((self.B, n, self.H, self.D), dtype=self.dtype)
        for j in range(n):
            p = m - n + j  # absolute position of the j-th visible row
            k[:, j] = self.k[layer, :, :, p % self.W, :]
            v[:, j] = self.v[layer, :, :, p % self.W, :]
        return k, v

    def write(self, layer: int, k_new, v_new):
        """Stage the row for absolute position ``t`` into slot ``t % W``.

        inference/kv_cache.py:44-51: input with ``shape[1] == 1`` is read as
        ``[B, 1, H, D]``; anything else as ``[B, H, 1, D]``.
        """
        k_new = np.asarray(k_new)
        v_new = np.asarray(v_new)
        if k_new.shape[1] == 1:
            k_new = np.swapaxes(k_new, 1, 2)
            v_new = np.swapaxes(v_new, 1, 2)
        i = self.t % self.W
        self.k[layer, :, :, i, :] = k_new[:, :, 0, :]
        self.v[layer, :, :, i, :] = v_new[:, :, 0, :]
        self.staged[layer] = True

    def advance(self):
        # inference/kv_cache.py:53-55
        self.t += 1
        self.staged = [False] * self.L

    def bulk_write_packed(self, kv, pos: int):
        """Store the last ``min(pos, W - 1)`` prompt positions; ``t = pos``.

        inference/kv_cache.py:57-68.  ``kv`` is ``[2, L, B, H, T, D]``.
        """
        kv = np.asarray(kv)
        r = min(pos, max(self.W - 1, 0))
        for p in range(pos - r, pos):
            self.k[:, :, :, p % self.W, :] = kv[0][:, :, :, p, :]
            self.v[:, :, :, p % self.W, :] = kv[1][:, :, :, p, :]
        self.t = pos
        self.staged = [False] * self.L
