"""Ring-buffer KV cache with the public surface of the reference's ``KVCache``
(inference/kv_cache.py:4-68): storage ``k, v [L, B, H, W, D]``, the token at
position ``p`` lives in slot ``p % W``, ``view`` returns the live rows in
chronological order, ``write`` stages the row of position ``t`` and ``advance``
moves on by one position.

``ring(layer)`` is an addition for the HIP decode kernel: it hands out the layer's
storage as it lies (slot order) so that a decode step reads the ring in place,
writes the new row itself, and no chronological copy is ever made.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch
from torch import Tensor


@dataclass
class RingContext:
    """Handle to one layer of a ``KVCache`` for the in-place decode path.

    ``k``/``v`` are the layer's ``[B, H, W, D]`` storage (views, not copies) and
    ``t`` the number of positions written so far; the row for position ``t``
    goes to slot ``t % W``.
    """
    cache: "KVCache"
    layer: int
    k: Tensor
    v: Tensor
    t: int
    W: int
    # one int32 on the GPU in which a step whose position lives in device memory reports what the
    # host cannot check beforehand (a position past the rotary tables); None = not wanted
    status: Optional[Tensor] = None

    def mark_written(self) -> None:
        self.cache._staged[self.layer] = True


class KVCache:
    """``t`` positions have been committed; a layer whose row for position ``t`` has been written
    but not yet committed is *staged* (``advance`` commits all layers at once)."""

    def __init__(self, L, B, H, W, D, device, dtype):
        self.L, self.B, self.H, self.W, self.D = L, B, H, W, D
        self.device, self.dtype = device, dtype
        self.k = torch.zeros((L, B, H, W, D), device=device, dtype=dtype)
        self.v = torch.zeros_like(self.k)
        self.t = 0
        self._staged = [False] * L

    def reset_history(self):
        # The reference allocates fresh zero tensors here (kv_cache.py:19-23); the storage is
        # reused instead so that a long-lived cache never reallocates.
        for store in (self.k, self.v):
            store.zero_()
        self.t = 0
        self._staged = [False] * self.L

    # -- reading -----------------------------------------------------------------------------
    def _live_rows(self, layer) -> Tuple[int, int]:
        """(first position, number of rows) that ``view`` shows: the newest ``min(written, W)``."""
        written = self.t + (1 if self._staged[layer] else 0)
        rows = min(written, self.W)
        return written - rows, rows

    def view(self, layer) -> Tuple[Tensor, Tensor]:
        """The live rows of a layer, oldest first, as ``[B, n, H, D]`` (``n = 0`` for an empty
        cache).  A run of slots that does not wrap is returned as a view; a run that wraps is
        the tail of the ring followed by its head (a copy)."""
        first, rows = self._live_rows(layer)
        lo = first % self.W if rows else 0
        hi = lo + rows
        out = []
        for store in (self.k[layer], self.v[layer]):          # [B, H, W, D]
            if hi <= self.W:
                run = store[:, :, lo:hi]
            else:
                run = torch.cat((store[:, :, lo:], store[:, :, :hi - self.W]), dim=2)
            out.append(run.transpose(1, 2))
        return out[0], out[1]

    def ring(self, layer) -> RingContext:
        """In-place handle for the decode kernel (no copy)."""
        return RingContext(self, layer, self.k[layer], self.v[layer], self.t, self.W)

    # -- writing -----------------------------------------------------------------------------
    def write(self, layer, k_new, v_new):
        """Stages the row of position ``t`` in slot ``t % W``.  A row may come as ``[B, 1, H, D]``
        or ``[B, H, 1, D]``; as in the reference, a size-1 second dim marks the former."""
        slot = self.t % self.W
        for store, row in ((self.k, k_new), (self.v, v_new)):
            if row.size(1) == 1:
                row = row.transpose(1, 2)
            store[layer, :, :, slot] = row[:, :, 0]
        self._staged[layer] = True

    def advance(self):
        """Commits the staged rows of all layers: position ``t`` is done."""
        self.t += 1
        self._staged = [False] * self.L

    def _prompt_runs(self, pos):
        """A prompt of ``pos`` tokens leaves room for the token that follows: only its last
        ``min(pos, W - 1)`` positions are kept.  Position p goes to slot ``p % W``, so the kept
        positions land in at most two runs of consecutive slots; returns ``(source, slots)``
        slice pairs (plain slice copies run several times faster than an indexed scatter)."""
        kept = min(pos, max(self.W - 1, 0))
        runs = []
        first = pos - kept
        while kept > 0:
            slot = first % self.W
            n = min(kept, self.W - slot)
            runs.append((slice(first, first + n), slice(slot, slot + n)))
            first, kept = first + n, kept - n
        return runs

    def bulk_write_packed(self, kv, pos):
        """Stores a prompt's keys and values from ``kv [2, L, B, H, T, D]`` and sets ``t = pos``."""
        for src, slots in self._prompt_runs(pos):
            self.k[:, :, :, slots].copy_(kv[0][:, :, :, src])
            self.v[:, :, :, slots].copy_(kv[1][:, :, :, src])
        self.t = pos
        self._staged = [False] * self.L

    def bulk_write_layer(self, layer, k, v, pos):
        """Per-layer form of ``bulk_write_packed`` for ``k, v [B, H, T, D]``; does not move ``t``."""
        for src, slots in self._prompt_runs(pos):
            self.k[layer][:, :, slots].copy_(k[:, :, src])
            self.v[layer][:, :, slots].copy_(v[:, :, src])
