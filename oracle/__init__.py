"""CPU oracle for Daisy's attention hot path (TEST INFRASTRUCTURE ONLY).

This package is a plain fp32 PyTorch/numpy restatement of the algorithms the
reference implements for the attention path.  It exists so the HIP kernels can
be checked against something that is obviously the same mathematics as the
reference; it is never the thing shipped or measured.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  Nothing under ``daisy_amd/`` imports it.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).

Pinning status (what independently checks each oracle function; the checks
live in ``tests/test_oracle_pins.py``):

* ``rope_tables`` / ``apply_rope``  -- closed-form invariants (position 0 is the
  identity, zero-frequency channels are untouched, pair norms are preserved,
  the rotated inner product depends only on the position difference, and the
  rotation direction is fixed by an explicit 2-D known answer).
* ``rms_norm``                      -- the library routine ``F.rms_norm``.
* ``build_attn_mask``               -- brute-force loops over (q, k) on tiny inputs.
* ``sdpa`` / ``windowed_attention`` -- the library routine
  ``F.scaled_dot_product_attention`` with an explicit additive mask, the
  ``is_causal=True`` special case, and per-row brute force.
* ``attn_prefill`` / ``attn_step``  -- the invariant "T steps == one prefill"
  used by the reference's own tests, plus per-token windowed brute force; their
  value-embedding mix by known answers (gate logit +30 -> v, -30 -> ve, and the
  reference's first-layer logit 0.3228 -> 0.58 v + 0.42 ve worked by hand).
* ``block_mask_dense``              -- torch's own ``BlockMask.from_kv_blocks`` built
  from block lists and expanded pair by pair with its ``mask_mod``.
* ``block_mask_cycle``              -- literal per-layer lists for 1, 2, 4, 5 and 8 layers.
* ``RingKVCache``                   -- the integer-valued scenarios of the
  reference's KV-cache tests (stored as data in ``tests/golden``).
* ``kda_gate``                      -- ``F.softplus`` / ``exp`` closed form.
* ``l2norm``                        -- hand-worked vectors ((3, 4) -> (0.6, 0.8)) and the
  epsilon's place inside the square root.
* ``short_conv`` / ``gated_rms_norm`` / ``kimi_layer_forward`` -- ``F.conv1d`` on an explicitly
  padded sequence + ``F.silu``, brute-force tap loops, "two calls with the carried window == one
  call", ``F.rms_norm`` with a weight times ``torch.sigmoid``.  PARITY UNPINNED against the
  absent flash-linear-attention modules they restate (see ``oracle/kimi.py``).
* ``kda_recurrent``                 -- closed forms (T=1, beta=0, g=0 cases),
  split-with-carried-state equivalence and an independent float64 loop.
  PARITY UNPINNED at one boundary: the third-party ``fla.ops.kda.chunk_kda``
  (flash-linear-attention, version not pinned by the reference, absent here)
  fixes conventions that are not visible in the reference tree -- the default
  ``scale`` (taken as Dk**-0.5), the L2-norm epsilon (taken as 1e-6 inside the
  square root) and its bf16 rounding points.  Those are explicit arguments here.
"""
from .attention import (  # noqa: F401
    rope_tables,
    apply_rope,
    rms_norm,
    build_attn_mask,
    doc_start_from_ids,
    block_mask_dense,
    block_mask_cycle,
    window_mask,
    sdpa,
    windowed_attention,
    windowed_attention_blockwise,
    calc_qkv,
    attn_prefill,
    attn_step,
)
from .kv_cache import RingKVCache  # noqa: F401
from .kda import kda_gate, kda_recurrent, l2norm  # noqa: F401
from .kimi import short_conv, gated_rms_norm, kimi_layer_forward  # noqa: F401
