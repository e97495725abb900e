"""Training-time block masks (models/daisy/daisy_core.py:182-229): the per-row lower bounds the
drop-in hands to the kernel describe exactly the set of (q, k) pairs the reference's BlockMask
construction keeps.  CPU only: the oracle restates the block lists, the product uses a closed form."""
import pytest
import torch

import oracle
from daisy_amd import build_block_window_masks


def _ids(T, p_eos, seed):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(2, 50, (T,), generator=g)
    ids[torch.rand(T, generator=g) < p_eos] = 1
    return ids


@pytest.mark.parametrize("T,block", [(1024, 128), (512, 64)])
@pytest.mark.parametrize("p_eos", [0.0, 0.002, 0.02, 0.3])
@pytest.mark.parametrize("w", [1, 2, 3, 5, 8])
def test_row_bounds_equal_the_block_lists(T, block, p_eos, w):
    ids = _ids(T, p_eos, seed=T + w + int(p_eos * 1000))
    dense = oracle.block_mask_dense(ids, w, eos_token_id=1, block=block)
    masks = build_block_window_masks(ids, w, 1, eos_token_id=1, block=block)
    assert len(masks) == 1 and masks[0].window is None
    lo = masks[0].doc_start.long()
    pos = torch.arange(T)
    mine = (pos[None, :] >= lo[:, None]) & (pos[None, :] <= pos[:, None])
    assert torch.equal(mine, dense)
    assert bool((lo[1:] >= lo[:-1]).all()), "lower bounds must not decrease (the kernel skips tiles by them)"


def test_document_boundaries_at_block_edges_and_single_document():
    T, block = 512, 128
    ids = torch.full((T,), 7)
    for eos_at in ([], [0], [128], [127, 128, 129], [255, 256], [511]):
        x = ids.clone()
        x[eos_at] = 1
        for w in (1, 2, 4):
            lo = build_block_window_masks(x, w, 1, eos_token_id=1, block=block)[0].doc_start.long()
            pos = torch.arange(T)
            mine = (pos[None, :] >= lo[:, None]) & (pos[None, :] <= pos[:, None])
            assert torch.equal(mine, oracle.block_mask_dense(x, w, 1, block)), (eos_at, w)


def test_long_short_cycle():
    ids = _ids(1024, 0.01, 3)
    for L in (1, 2, 4, 5, 8, 12):
        masks = build_block_window_masks(ids, 6, L, eos_token_id=1)
        assert len(masks) == L
        widths = oracle.block_mask_cycle(L, 6)
        long_m, short_m = masks[0], (masks[1] if L > 2 else None)
        for m, wd in zip(masks, widths):
            assert m is (long_m if wd == 6 else short_m)
        assert masks[-1] is long_m


def test_length_must_be_a_multiple_of_the_block():
    with pytest.raises(Exception, match="divisible"):
        build_block_window_masks(torch.zeros(100, dtype=torch.long), 2, 1, eos_token_id=1)
