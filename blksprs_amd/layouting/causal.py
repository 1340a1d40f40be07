"""Layouts and compact masks of causal (optionally windowed) self-attention over padded sequences.

Same functions, results and error types as the reference (blksprs/layouting/causal.py:16-252).  These are
descriptions of sequence structure, a few kilobytes of boolean data, computed with torch on whatever device
the lengths live on; the attention kernels themselves can evaluate the same predicate natively from
``causal_lengths`` and then need no mask at all.
"""

from collections.abc import Sequence

import torch
from torch import Tensor

from ..utils.blksprs_tensor import BlksprsTensor


def _lengths_1d(valid_lengths, device=None) -> Tensor:
    """The valid lengths as a one-dimensional int64 tensor (blksprs/layouting/causal.py:222-233)."""
    t = torch.as_tensor(valid_lengths, device=device)
    if t.dim() != 1:
        raise ValueError("valid_lengths must be one-dimensional")
    if t.dtype == torch.bool or t.is_floating_point():
        raise TypeError("valid_lengths must use an integer dtype")
    if bool((t < 0).any()):
        raise ValueError("valid_lengths must be non-negative")
    return t.long()


def _check_block_size(sparsity_block_size) -> None:
    if isinstance(sparsity_block_size, bool) or not isinstance(sparsity_block_size, int):
        raise TypeError("sparsity_block_size must be an integer")
    if sparsity_block_size < 1:
        raise ValueError("sparsity_block_size must be positive")


def _check_window(window_size) -> None:
    if isinstance(window_size, bool) or not isinstance(window_size, int):
        raise TypeError("window_size must be an integer")
    if window_size < 1:
        raise ValueError("window_size must be positive")


def _blocks_needed(lengths: Tensor, sbs: int) -> Tensor:
    return (lengths + (sbs - 1)).div(sbs, rounding_mode="floor")


def build_causal_self_attention_layout(valid_lengths: Tensor | Sequence[int], sparsity_block_size: int) -> Tensor:
    """Lower-triangular block layout of padded causal self-attention.

    Block ``(q, k)`` of batch entry ``b`` is active when ``k <= q`` and both block rows reach into the first
    ``valid_lengths[b]`` positions; the grid has ``ceil(max(valid_lengths) / sparsity_block_size)`` blocks per
    side.  A partial last block stays active (the mask of ``build_causal_self_attention_mask`` refines it).

    Returns:
        Tensor: bool ``(B, n, n)``, contiguous.

    """
    lengths = _lengths_1d(valid_lengths)
    _check_block_size(sparsity_block_size)
    n = 0 if lengths.numel() == 0 else -(-int(lengths.max()) // sparsity_block_size)
    if n == 0:
        return torch.zeros((lengths.numel(), 0, 0), dtype=torch.bool, device=lengths.device)
    idx = torch.arange(n, device=lengths.device)
    inside = idx[None, :] < _blocks_needed(lengths, sparsity_block_size)[:, None]      # (B, n)
    causal = idx[:, None] >= idx[None, :]                                               # (n, n): query >= key
    return (inside[:, :, None] & inside[:, None, :] & causal[None]).contiguous()


def _mask_and_layout(valid_lengths, attention_layout: Tensor, sbs: int, window_size: int | None):
    """Shared body of the two mask builders (blksprs/layouting/causal.py:85-178)."""
    lengths = _lengths_1d(valid_lengths, device=attention_layout.device)
    _check_block_size(sbs)
    if attention_layout.dtype != torch.bool:
        raise TypeError("attention_layout must have dtype torch.bool")
    if attention_layout.dim() != 3:
        raise ValueError("attention_layout must have shape (batch, query_blocks, key_blocks)")
    if not attention_layout.is_contiguous():
        raise ValueError("attention_layout must be contiguous")
    if attention_layout.size(0) != lengths.numel():
        raise ValueError("valid_lengths and attention_layout must have the same batch size")
    if attention_layout.size(1) != attention_layout.size(2):
        raise ValueError("causal self-attention requires a square attention_layout")
    n = attention_layout.size(1)
    longest = int(lengths.max()) if lengths.numel() else 0
    if n != -(-longest // sbs):
        raise ValueError("attention_layout does not match the longest valid length")
    if bool((attention_layout & ~build_causal_self_attention_layout(lengths, sbs)).any()):
        raise ValueError("attention_layout contains blocks outside the valid causal prefix.")

    dev = attention_layout.device
    no_mask = torch.empty((0, sbs, sbs), dtype=torch.bool, device=dev)
    if n == 0:
        return BlksprsTensor.wrap(no_mask), torch.zeros_like(attention_layout)

    # blocks that can hold a masked score: the diagonal (future keys), the far edge of the window, and the
    # whole row of a partial last query block (its padding rows are masked in every key block)
    idx = torch.arange(n, device=dev)
    q_blk, k_blk = idx[:, None], idx[None, :]
    candidates = (q_blk == k_blk)
    if window_size is not None:
        candidates = candidates | ((q_blk - k_blk) == -(-(window_size - 1) // sbs))
    last = _blocks_needed(lengths, sbs) - 1                                             # (B,)
    partial = (lengths % sbs) != 0
    ragged_row = partial[:, None, None] & (q_blk[None] == last[:, None, None]) & (k_blk[None] <= last[:, None, None])
    mask_layout = (attention_layout & (candidates[None] | ragged_row)).contiguous()

    where = mask_layout.nonzero()
    if where.size(0) == 0:
        return BlksprsTensor.wrap(no_mask), mask_layout
    offs = torch.arange(sbs, device=dev)
    q_pos = (where[:, 1] * sbs)[:, None, None] + offs[None, :, None]                    # (nnz, sbs, 1)
    k_pos = (where[:, 2] * sbs)[:, None, None] + offs[None, None, :]                    # (nnz, 1, sbs)
    length = lengths[where[:, 0]][:, None, None]
    mask = (k_pos > q_pos) | (q_pos >= length) | (k_pos >= length)
    if window_size is not None:
        mask = mask | (q_pos - k_pos > window_size - 1)
    return BlksprsTensor.wrap(mask.contiguous()), mask_layout


def build_causal_self_attention_mask(valid_lengths: Tensor | Sequence[int], attention_layout: Tensor,
                                     sparsity_block_size: int) -> tuple[BlksprsTensor, Tensor]:
    """Compact causal / padding mask of a causal attention layout (``True`` = score ignored, the convention of
    ``flash_attention``).  Its layout holds only the blocks that can contain a masked score: the diagonal
    blocks and, where the last query block of a sequence is partial, that block row.

    Returns:
        tuple[BlksprsTensor, Tensor]: ``(attention_mask, sparsity_layout_mask)``.

    """
    return _mask_and_layout(valid_lengths, attention_layout, sparsity_block_size, None)


def build_causal_window_self_attention_layout(valid_lengths: Tensor | Sequence[int], sparsity_block_size: int,
                                              window_size: int) -> Tensor:
    """Causal block layout restricted to the last ``window_size`` tokens (the current token counts, so 1 is
    self-attention only).  Blocks the window only touches stay active; the window mask refines them."""
    _check_window(window_size)
    layout = build_causal_self_attention_layout(valid_lengths, sparsity_block_size)
    idx = torch.arange(layout.size(1), device=layout.device)
    near = (idx[:, None] - idx[None, :]) <= -(-(window_size - 1) // sparsity_block_size)
    return (layout & near[None]).contiguous()


def build_causal_window_self_attention_mask(valid_lengths: Tensor | Sequence[int], attention_layout: Tensor,
                                            sparsity_block_size: int, window_size: int) -> tuple[BlksprsTensor, Tensor]:
    """Compact causal / padding / window mask for local causal attention."""
    _check_window(window_size)
    return _mask_and_layout(valid_lengths, attention_layout, sparsity_block_size, window_size)
