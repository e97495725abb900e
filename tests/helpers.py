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


def flex_block_mask(ids: torch.Tensor, window_blocks: int, eos: int, block: int = 128):
    """A ``torch.nn.attention.flex_attention.BlockMask`` for document-causal attention with a window
    counted in key blocks, assembled the way the reference's training forward assembles its masks
    (models/daisy/daisy_core.py:182-221): per query block the list of *full* key blocks (strictly
    earlier, both blocks inside one document) and of *partial* ones (touching causally and by
    document), each ordered from the most recent block backwards, cut to ``window - 1`` full blocks
    and ``max(window - n_full, 1)`` partial ones; pairs inside partial blocks are decided by
    ``mask_mod(q, k) = q >= k and same document``.  Written with explicit loops over blocks.
    """
    from torch.nn.attention.flex_attention import BlockMask
    ids = ids.reshape(-1)
    T = ids.numel()
    nb = T // block
    docs = torch.cumsum((ids == eos).to(torch.int64), 0)
    first_doc, last_doc = docs.view(nb, block)[:, 0], docs.view(nb, block)[:, -1]
    n_full = torch.zeros(nb, dtype=torch.int32)
    n_part = torch.zeros(nb, dtype=torch.int32)
    full_idx = torch.zeros(nb, nb, dtype=torch.int32)
    part_idx = torch.zeros(nb, nb, dtype=torch.int32)
    for i in range(nb):
        full, part = [], []
        for j in range(nb - 1, -1, -1):                       # most recent first
            touches = j <= i and first_doc[i] <= last_doc[j] and last_doc[i] >= first_doc[j]
            whole = j < i and first_doc[i] == last_doc[j] and last_doc[i] == first_doc[j]
            if touches and whole:
                full.append(j)
            elif touches:
                part.append(j)
        rest_f = [j for j in range(nb - 1, -1, -1) if j not in full]
        rest_p = [j for j in range(nb - 1, -1, -1) if j not in part]
        full_idx[i] = torch.tensor(full + rest_f, dtype=torch.int32)
        part_idx[i] = torch.tensor(part + rest_p, dtype=torch.int32)
        n_full[i] = min(len(full), window_blocks - 1)
        n_part[i] = min(len(part), max(window_blocks - len(full), 1))

    def document_causal(b, h, q_idx, kv_idx):
        return (q_idx >= kv_idx) & (docs[q_idx] == docs[kv_idx])

    return BlockMask.from_kv_blocks(n_part[None, None], part_idx[None, None], n_full[None, None], full_idx[None, None],
                                    BLOCK_SIZE=block, mask_mod=document_causal)


def block_mask_pairs(bm) -> torch.Tensor:
    """Boolean ``[T, T]``: the (query, key) pairs a ``BlockMask`` lets ``flex_attention`` see -- every
    pair of a listed full block, the pairs that ``mask_mod`` keeps of a listed partial block."""
    qb, kb = bm.BLOCK_SIZE
    T = bm.seq_lengths[0]
    allowed = torch.zeros(T, T, dtype=torch.bool)
    num_p, idx_p = bm.kv_num_blocks[0, 0], bm.kv_indices[0, 0]
    num_f, idx_f = bm.full_kv_num_blocks[0, 0], bm.full_kv_indices[0, 0]
    zero = torch.zeros((), dtype=torch.long)
    for i in range(idx_p.shape[0]):
        qs = torch.arange(i * qb, min((i + 1) * qb, T))
        for j in idx_f[i, :int(num_f[i])].tolist():
            allowed[i * qb:(i + 1) * qb, j * kb:(j + 1) * kb] = True
        for j in idx_p[i, :int(num_p[i])].tolist():
            ks = torch.arange(j * kb, min((j + 1) * kb, T))
            allowed[qs[0]:qs[-1] + 1, ks[0]:ks[-1] + 1] = bm.mask_mod(zero, zero, qs[:, None], ks[None, :])
    return allowed
