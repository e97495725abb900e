"""Training-time block masks (models/daisy/daisy_core.py:182-229): the per-row lower bounds the
drop-in hands to the kernel describe exactly the set of (q, k) pairs the reference's BlockMask
construction keeps.  CPU only: the oracle restates the block lists, the product uses a closed form."""
import pytest
import torch

import oracle
from daisy_amd import build_block_window_masks
from daisy_amd.attention import block_mask_to_window, dense_mask_to_window
from helpers import block_mask_pairs, flex_block_mask


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


@pytest.mark.parametrize("p_eos", [0.0, 0.01, 0.1])
@pytest.mark.parametrize("w", [1, 2, 3, 4])
def test_oracle_block_mask_equals_the_library_block_mask(p_eos, w):
    """Pins oracle.block_mask_dense against torch's own BlockMask.from_kv_blocks, expanded pair by pair."""
    T, block = 512, 64
    ids = _ids(T, p_eos, seed=17 + w)
    bm = flex_block_mask(ids, w, eos=1, block=block)
    assert torch.equal(oracle.block_mask_dense(ids, w, eos_token_id=1, block=block), block_mask_pairs(bm))


@pytest.mark.parametrize("p_eos", [0.0, 0.02, 0.2])
@pytest.mark.parametrize("w", [1, 2, 5])
def test_a_library_block_mask_converts_to_the_same_row_bounds(p_eos, w):
    """What CausalSelfAttention.forward does with the BlockMask the reference's training forward passes."""
    T, block = 512, 64
    ids = _ids(T, p_eos, seed=29 + w)
    bm = flex_block_mask(ids, w, eos=1, block=block)
    mask = block_mask_to_window(bm, pairs_per_pass=7)
    lo = mask.doc_start.long()
    assert mask.window is None and lo.dtype == torch.int64 and mask.doc_start.dtype == torch.int32
    pos = torch.arange(T)
    mine = (pos[None, :] >= lo[:, None]) & (pos[None, :] <= pos[:, None])
    assert torch.equal(mine, block_mask_pairs(bm))
    assert torch.equal(mask.doc_start, build_block_window_masks(ids, w, 1, eos_token_id=1, block=block)[0].doc_start)


def test_block_masks_that_are_not_causal_bands_are_refused():
    from torch.nn.attention.flex_attention import create_block_mask
    T = 256
    with pytest.raises(ValueError, match="one run of keys"):      # bidirectional: keys after the query
        block_mask_to_window(create_block_mask(lambda b, h, q, k: (q - k).abs() < 40, 1, 1, T, T, device="cpu", BLOCK_SIZE=64))
    with pytest.raises(ValueError, match="one run of keys"):      # a hole in the middle of the run
        block_mask_to_window(create_block_mask(lambda b, h, q, k: (q >= k) & ((q - k) % 2 == 0), 1, 1, T, T, device="cpu", BLOCK_SIZE=64))
    ok = block_mask_to_window(create_block_mask(lambda b, h, q, k: (q >= k) & (q - k < 100), 1, 1, T, T, device="cpu", BLOCK_SIZE=64))
    assert ok.doc_start.tolist() == [max(0, q - 99) for q in range(T)]


def test_dense_masks_with_a_bound_that_moves_backwards_are_refused():
    T = 12
    pos = torch.arange(T)
    lo = torch.tensor([0, 0, 1, 2, 1, 2, 3, 4, 5, 6, 7, 8])      # row 4 sees one key more than row 3 allows
    dense = torch.where((pos[None, :] >= lo[:, None]) & (pos[None, :] <= pos[:, None]), 0.0, float("-inf"))[None, None]
    with pytest.raises(ValueError, match="decreases"):
        dense_mask_to_window(dense)
    lo[4] = 2
    dense = torch.where((pos[None, :] >= lo[:, None]) & (pos[None, :] <= pos[:, None]), 0.0, float("-inf"))[None, None]
    assert dense_mask_to_window(dense).doc_start.tolist() == lo.tolist()


def test_long_short_cycle_literal_lists():
    """models/daisy/daisy_core.py:224-229: long, short, short, short, ... and the last layer long."""
    L_, S_ = 6, 3
    want = {1: [L_], 2: [L_, L_], 4: [L_, S_, S_, L_], 5: [L_, S_, S_, S_, L_], 8: [L_, S_, S_, S_, L_, S_, S_, L_]}
    for n_layers, widths in want.items():
        assert oracle.block_mask_cycle(n_layers, 6) == widths
    assert oracle.block_mask_cycle(4, 7) == [7, 3, 3, 7]          # short = long // 2


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
