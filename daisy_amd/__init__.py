"""MI355X-native attention hot path for Daisy.

Hand-written gfx950 HIP kernels (``daisy_amd/csrc``, C ABI in
``include/daisy_hip.h``) behind the reference's own Python interfaces:
``CausalSelfAttention``, ``KVCache``, ``Generator``, ``chunk_kda`` and
``fused_kda_gate``.
"""
from .attention import (CausalSelfAttention, Rotary, WindowMask, build_block_window_masks,  # noqa: F401
                        build_window_mask, dense_mask_to_window, doc_start_from_ids)
from . import core  # noqa: F401
from .attention_kimi import KimiLinearSelfAttention  # noqa: F401
from .functional import norm  # noqa: F401
from .generate import Generator  # noqa: F401
from .kda import chunk_kda, fused_kda_gate, fused_recurrent_kda  # noqa: F401
from .kv_cache import KVCache, RingContext  # noqa: F401

__all__ = [
    "CausalSelfAttention", "Rotary", "WindowMask", "build_window_mask", "build_block_window_masks", "dense_mask_to_window",
    "doc_start_from_ids", "norm", "Generator", "chunk_kda", "fused_kda_gate", "fused_recurrent_kda", "KVCache", "RingContext", "core", "KimiLinearSelfAttention",
]
