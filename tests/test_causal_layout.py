"""Causal layout and mask builders (pure torch, run on the CPU): the known answers the reference's own tests
hold (test/cases/test_causal_layout.py:12-55), and brute force against the token-level oracle."""

import numpy as np
import pytest
import torch

from blksprs_amd.layouting import (build_causal_self_attention_layout, build_causal_self_attention_mask,
                                   build_causal_window_self_attention_layout,
                                   build_causal_window_self_attention_mask)
from oracle import blksprs_oracle as orc


def test_layout_tracks_each_valid_prefix():
    layout = build_causal_self_attention_layout(torch.tensor([1, 17, 32]), 16)
    assert layout.dtype is torch.bool and layout.shape == (3, 2, 2) and layout.is_contiguous()
    assert torch.equal(layout[0], torch.tensor([[True, False], [False, False]]))
    assert torch.equal(layout[1], torch.tensor([[True, False], [True, True]]))
    assert torch.equal(layout[2], torch.tensor([[True, False], [True, True]]))


def test_mask_is_compact_and_masks_future_and_padding():
    layout = build_causal_self_attention_layout(torch.tensor([17]), 16)
    mask, mask_layout = build_causal_self_attention_mask(torch.tensor([17]), layout, 16)
    assert torch.equal(mask_layout[0], torch.tensor([[True, False], [True, True]]))
    assert mask.shape == (3, 16, 16) and mask.dtype is torch.bool
    assert not mask[0, 15, 0] and mask[0, 0, 1]            # first diagonal block: strictly upper triangle only
    assert not mask[1, 0, 0] and mask[1, 1, 0]             # off-diagonal block of the partial query block: padding rows
    assert not mask[2, 0, 0] and mask[2, 0, 1] and mask[2, 1, 0]  # partial diagonal block: future and padding


def test_window_mask_refines_the_boundary_block():
    layout = build_causal_window_self_attention_layout(torch.tensor([32]), 16, 17)
    mask, mask_layout = build_causal_window_self_attention_mask(torch.tensor([32]), layout, 16, 17)
    assert torch.equal(layout[0], torch.tensor([[True, False], [True, True]]))
    assert torch.equal(mask_layout[0], torch.tensor([[True, False], [True, True]]))
    assert not mask[1, 0, 0] and mask[1, 15, 0]            # token 16 reaches back 16 tokens, token 31 does not reach token 0


@pytest.mark.parametrize("lengths", [torch.tensor([-1]), torch.ones((1, 1), dtype=torch.long)])
def test_invalid_lengths_are_rejected(lengths):
    with pytest.raises((TypeError, ValueError)):
        build_causal_self_attention_layout(lengths, 16)


def test_argument_errors():
    layout = build_causal_self_attention_layout([20], 8)
    with pytest.raises(TypeError):
        build_causal_self_attention_layout(torch.tensor([1.0]), 8)
    with pytest.raises(TypeError):
        build_causal_self_attention_layout([4], True)
    with pytest.raises(ValueError):
        build_causal_self_attention_layout([4], 0)
    with pytest.raises(TypeError):
        build_causal_self_attention_mask([20], layout.int(), 8)
    with pytest.raises(ValueError, match="same batch size"):
        build_causal_self_attention_mask([20, 20], layout, 8)
    with pytest.raises(ValueError, match="longest valid length"):
        build_causal_self_attention_mask([40], layout, 8)
    with pytest.raises(ValueError, match="square"):
        build_causal_self_attention_mask([20], torch.ones((1, 3, 2), dtype=torch.bool), 8)
    with pytest.raises(ValueError, match="contiguous"):
        build_causal_self_attention_mask([20], torch.ones((1, 3, 6), dtype=torch.bool)[:, :, ::2], 8)
    with pytest.raises(ValueError, match="outside the valid causal prefix"):
        build_causal_self_attention_mask([20], torch.ones((1, 3, 3), dtype=torch.bool), 8)
    with pytest.raises(TypeError):
        build_causal_window_self_attention_layout([20], 8, 2.0)
    with pytest.raises(ValueError):
        build_causal_window_self_attention_layout([20], 8, 0)
    with pytest.raises(ValueError):
        build_causal_window_self_attention_mask([20], layout, 8, -1)


@pytest.mark.parametrize("window", [None, 1, 5, 8, 9, 23])
@pytest.mark.parametrize("lengths", [[0], [1], [8], [9, 24, 17], [31, 2], [16, 16]])
def test_layout_and_mask_against_the_token_level_oracle(lengths, window):
    """The dense token mask implied by (layout, compact mask) equals the token-level predicate wherever the
    layout is active, inactive blocks are exactly the blocks in which every score is ignored or that lie above
    the diagonal / outside the window band."""
    s = 8
    if window is None:
        layout = build_causal_self_attention_layout(lengths, s)
        mask, mask_layout = build_causal_self_attention_mask(lengths, layout, s)
    else:
        layout = build_causal_window_self_attention_layout(lengths, s, window)
        mask, mask_layout = build_causal_window_self_attention_mask(lengths, layout, s, window)
    assert np.array_equal(layout.numpy(), orc.causal_layout(lengths, s, window))
    assert np.array_equal(mask_layout.numpy(), orc.causal_mask_layout(lengths, layout.numpy(), s, window))
    n = layout.size(1)
    assert mask.shape[0] == int(mask_layout.sum()) and not bool((mask_layout & ~layout).any())
    where = mask_layout.nonzero().tolist()
    for b, length in enumerate(lengths):
        token = orc.causal_token_mask(length, n * s, window)
        for q in range(n):
            for k in range(n):
                want = token[q * s:(q + 1) * s, k * s:(k + 1) * s]
                if [b, q, k] in where:
                    assert np.array_equal(mask[where.index([b, q, k])].numpy(), want)
                elif layout[b, q, k]:
                    # an active block without a mask block masks nothing -- except the one block the reference
                    # leaves unrefined: one offset nearer than the window's far block, when the window does not
                    # end on a block boundary
                    unrefined = window is not None and (window - 1) % s != 0 and q - k == -(-(window - 1) // s) - 1
                    assert unrefined or not want.any()
                else:
                    assert want.all()           # a dropped block holds no score that counts
