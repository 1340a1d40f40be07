"""Shared helpers of the GPU parity tests."""

import numpy as np
import torch
from torch import Tensor

from oracle import blksprs_oracle as orc


def rand_layout(shape, density, seed, ensure_rows=False):
    g = torch.Generator().manual_seed(seed)
    return orc.random_layout(shape, density, g, ensure_rows=ensure_rows)


def rand_blocks(n, sbs, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((n, sbs, sbs), generator=g) * scale).to(dtype)


def assert_close(got, expected, tol, what=""):
    """allclose with rtol = atol = tol, reporting where the worst element is."""
    got64, exp64 = got.detach().double().cpu(), expected.detach().double().cpu()
    assert got64.shape == exp64.shape, f"{what}: shape {tuple(got64.shape)} vs {tuple(exp64.shape)}"
    if got64.numel() == 0:
        return
    both_nan = torch.isnan(got64) & torch.isnan(exp64)
    err = (got64 - exp64).abs()
    err[both_nan] = 0
    bound = tol + tol * exp64.abs()
    bad = ~(err <= bound) & ~both_nan
    if bad.any():
        idx = torch.nonzero(bad)
        worst = int(torch.argmax(torch.where(bad, err - bound, torch.zeros_like(err)).reshape(-1)))
        pos = np.unravel_index(worst, tuple(got64.shape))
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{got64.numel()} elements off (tol {tol}); worst at {pos}: "
            f"got {got64[pos].item()!r} expected {exp64[pos].item()!r}; first bad {idx[0].tolist()}")


# ---------------------------------------------------------------------------------------------------------------
# The work orders of the matmul kernels, restated in torch: what the device builders are held to, bit for bit.

SUPER_TILE = 16
N_XCD = 8
ROWS_DOWNWARD = 1 << 30  # BSA_ROWS_DOWNWARD


def expected_block_order(layout_indices: Tensor, n_rows: int, n_cols: int) -> Tensor:
    """Work order of the output blocks of a layout with ``n_rows`` x ``n_cols`` blocks per batch entry: 16 x 16
    super-tiles of the block grid, columns of super-tiles fastest, so that the blocks in flight on one L2 share
    x row panels and y column panels.  A restatement in torch of what ``bsa_lut_block_order`` builds on the device."""
    b, i, j = layout_indices[:, 0], layout_indices[:, 1], layout_indices[:, 2]
    t = SUPER_TILE
    n_i = max(-(-n_rows // t), 1)
    n_j = max(-(-n_cols // t), 1)
    key = ((b * n_i + i // t) * n_j + j // t) * (t * t) + (i % t) * t + (j % t)
    return torch.argsort(key, stable=True).to(torch.int32)


def expected_row_work_table(pair_offsets: Tensor, row_offsets_o: Tensor, rows_per_batch: int, parts_log2: int,
                    pair_up: bool = False, max_work: int | None = None, sweep: int = 0) -> Tensor:
    """Order in which the row kernel hands parts of output block rows to workgroups: int32 entries
    ``row << parts_log2 | part``, -1 for nothing.  A restatement in torch of what ``bsa_lut_row_work_table`` builds
    on the device (runs on CPU tensors as well).

    Workgroup ``g`` runs on XCD ``g % 8``.  Every XCD gets one contiguous eighth of the rows (so the rows in
    flight on one L2 belong to the same batch entry and stream through the same y blocks), and walks it batch
    entry by batch entry, part by part, rows with the most (x, y) pairs first, so that the last workgroups of a
    launch are the short ones.  The k-th item of eighth c sits at position 8 k + c; eighths with a row less end
    in an empty entry.  With ``pair_up`` the rows of a batch entry alternate longest, shortest, second longest,
    second shortest, ...: a workgroup that takes two consecutive entries of its XCD's list then has about the
    same work as every other one, the workgroups of an XCD start and end their rows of one batch entry together
    (they stream through the same y blocks at the same time), and a launch ends without a tail of short rows.
    With ``sweep`` > 0 the items of one (XCD, batch entry, part) group alternate their direction every ``sweep``
    items: the first ``sweep`` walk their columns upward, the next ``sweep`` (which start as those end, on the
    same compute units) downward, and so on: a part that starts finds the y blocks its predecessors read last
    still in the L2.
    ``max_work`` is a bound on the pairs of one row that the caller knows without asking the device (inner
    blocks times output columns); without it the largest count is read back, which waits for the stream.
    """
    n_rows = row_offsets_o.numel() - 1
    parts = 1 << parts_log2
    device = row_offsets_o.device
    if n_rows == 0:
        return torch.empty(0, dtype=torch.int32, device=device)
    ends = pair_offsets[row_offsets_o.long()]
    work = (ends[1:] - ends[:-1]).long()
    small, extra = divmod(n_rows, N_XCD)
    # chunk c holds small + 1 rows for c < extra and small rows after that: plain arithmetic, nothing is copied
    # to the device
    all_rows = torch.arange(n_rows, device=device)
    long_rows = extra * (small + 1)
    chunk_of_row = torch.where(all_rows < long_rows, all_rows // (small + 1),
                               extra + (all_rows - long_rows) // max(small, 1))
    rows = all_rows.repeat_interleave(parts)
    part = torch.arange(parts, device=device).repeat(n_rows)
    entry = rows // max(rows_per_batch, 1)
    n_entries = n_rows // max(rows_per_batch, 1) + 1
    heaviest = int(work.max()) if max_work is None else int(max_work)
    key = ((chunk_of_row[rows] * n_entries + entry) * parts + part) * (heaviest + 1) + (heaviest - work[rows])
    by_chunk = torch.argsort(key, stable=True)  # chunk-major, batch entry, part, work descending
    # position of every item inside its (chunk, batch entry, part) group, and the group's size (the number of
    # groups is known here, so nothing is read back)
    group = (key // (heaviest + 1))[by_chunk]
    sizes_g = torch.zeros(N_XCD * n_entries * parts, dtype=torch.int64, device=device)
    sizes_g.scatter_add_(0, group, torch.ones_like(group))
    starts = torch.cumsum(sizes_g, 0) - sizes_g
    rank = torch.arange(rows.numel(), device=device) - starts[group]
    if pair_up:
        # within a group: longest, shortest, second longest, second shortest, ...
        m = sizes_g[group]
        spot = torch.where(rank < (m + 1) // 2, 2 * rank, 2 * (m - 1 - rank) + 1)
        reordered = torch.empty_like(by_chunk)
        reordered[starts[group] + spot] = by_chunk
        by_chunk = reordered
    chunk = chunk_of_row[rows][by_chunk]
    first_of_chunk = (chunk * small + torch.clamp(chunk, max=extra)) * parts
    within = torch.arange(rows.numel(), device=device) - first_of_chunk
    table = torch.full(((small + (extra > 0)) * parts * N_XCD,), -1, dtype=torch.int32, device=device)
    items = (rows[by_chunk] << parts_log2) | part[by_chunk]
    if sweep > 0:
        items = items | (((rank // sweep) & 1) * ROWS_DOWNWARD)
    table[within * N_XCD + chunk] = items.to(torch.int32)
    return table
