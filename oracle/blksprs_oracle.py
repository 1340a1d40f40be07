"""CPU restatement of the reference's block-sparse compute path.

TEST INFRASTRUCTURE ONLY.  Imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported baseline; the product
(``blksprs_amd``) never imports, calls or falls back to anything in this file.

Integer tables are numpy, floating-point operators are dense-masked torch on the CPU.
Every function names the reference lines it restates (paths relative to the
FelixSchoen/blksprs checkout).  How each one is pinned (brute force on tiny inputs,
closed forms, torch library routines, known answers held by the reference's tests)
is listed in ``tests/test_oracle_pins.py``; every function below has at least one
such pin, none is "parity unpinned".
"""

import math

import numpy as np
import torch

# --------------------------------------------------------------------------- lookup tables (integer, exact)


def packed_indices(layout) -> np.ndarray:
    """blksprs/utils/tools.py:38-57: ``where(l == 1, cumsum(l) - 1, -1)`` over the flattened layout, int64."""
    flat = np.asarray(layout).reshape(-1).astype(np.int64)
    return np.where(flat == 1, np.cumsum(flat) - 1, -1).astype(np.int64)


def layout_indices(layout) -> np.ndarray:
    """blksprs/utils/tools.py:33-35: ``nonzero(layout)`` as int64 ``[nnz, 3]`` in row-major order."""
    return np.argwhere(np.asarray(layout) != 0).astype(np.int64).reshape(-1, 3)


def n_sparse_blocks(layout) -> int:
    """blksprs/ops/conversion.py:286-288: the block count, summed in int64."""
    return int(np.asarray(layout).astype(np.int64).sum())


def segmented_indices(layout):
    """blksprs/ops/flash_attention.py:1923-1949: CSR adjacency ``(indices, offsets, max_per_row)``.

    ``layout`` is ``(B, rows, cols)``; offsets has ``B * rows + 1`` int32 entries starting at 0; indices are
    the active column ids row by row; empty or all-zero layouts give ``(empty, zeros, 1)``.
    """
    lay = np.asarray(layout).astype(np.int64)
    B, R, C = lay.shape
    counts = lay.sum(axis=2).reshape(-1)
    zeros = np.zeros(B * R + 1, dtype=np.int32)
    if counts.size == 0 or counts.max() == 0:
        return np.empty(0, dtype=np.int32), zeros, 1
    offsets = zeros.copy()
    offsets[1:] = np.cumsum(counts)
    indices = np.argwhere(lay.reshape(B * R, C) != 0)[:, 1].astype(np.int32)
    return indices, offsets, int(counts.max())


def segmented_index_dtype(n_active_blocks: int, n_blocks_col: int):
    """blksprs/ops/flash_attention.py:1952-1957."""
    limit = 2_147_483_647
    return np.int64 if (n_active_blocks > limit or n_blocks_col - 1 > limit) else np.int32


def sorted_packed_indices(layout):
    """blksprs/ops/softmax.py:652-666: per-row descending sort of the packed indices and
    ``max_blocks_line = ceil_pow2(max(longest row, 2))``."""
    lay = np.asarray(layout)
    packed = packed_indices(lay).reshape(lay.shape)
    srt = -np.sort(-packed, axis=-1)
    longest = int((srt.reshape(-1, lay.shape[-1]) != -1).sum(axis=-1).max()) if srt.size else 0
    longest = max(longest, 2)
    return srt.reshape(-1), 1 << (longest - 1).bit_length()


def layout_matmul(layout_x, layout_y) -> np.ndarray:
    """blksprs/layouting/sparsity_layout.py:244-258: boolean block product."""
    lx = np.asarray(layout_x).astype(np.int64)
    ly = np.asarray(layout_y).astype(np.int64)
    return np.einsum("bik,bkj->bij", lx, ly) > 0


def build_sparsity_layout(x, sparsity_block_size: int) -> np.ndarray:
    """blksprs/layouting/sparsity_layout.py:17-109: block (r, c) of batch entry b is active where any of its
    elements compares unequal to zero (``blk_x != 0``, :100), so NaN activates a block and -0.0 does not."""
    x = torch.as_tensor(x).detach().cpu()
    s = sparsity_block_size
    B, R, C = x.size(0), x.size(1) // s, x.size(2) // s
    return (x.reshape(B, R, s, C, s) != 0).any(dim=4).any(dim=2).numpy()


def causal_token_mask(valid_length: int, padded_length: int, window_size=None) -> np.ndarray:
    """Token-level statement of blksprs/layouting/causal.py:158-172: score (q, k) is ignored when the key lies
    in the future, when either position is padding, or (windowed) when the key is ``window_size`` or more
    tokens back.  bool ``(padded_length, padded_length)``, True = ignored.  Plain loops."""
    m = np.zeros((padded_length, padded_length), dtype=bool)
    for q in range(padded_length):
        for k in range(padded_length):
            ignored = k > q or q >= valid_length or k >= valid_length
            if window_size is not None and q - k > window_size - 1:
                ignored = True
            m[q, k] = ignored
    return m


def causal_layout(valid_lengths, sparsity_block_size: int, window_size=None) -> np.ndarray:
    """blksprs/layouting/causal.py:16-51 and :181-203 from the token-level mask: a block is active when
    k_block <= q_block, both block rows reach into the valid prefix and (windowed) the block offset does not
    exceed ceil((window_size - 1) / block size)."""
    s = sparsity_block_size
    lengths = [int(v) for v in valid_lengths]
    n = (max(lengths, default=0) + s - 1) // s
    out = np.zeros((len(lengths), n, n), dtype=bool)
    for b, length in enumerate(lengths):
        used = (length + s - 1) // s
        for q in range(n):
            for k in range(n):
                ok = k <= q and q < used and k < used
                if window_size is not None and q - k > (window_size - 1 + s - 1) // s:
                    ok = False
                out[b, q, k] = ok
    return out


def causal_mask_layout(valid_lengths, attention_layout, sparsity_block_size: int, window_size=None) -> np.ndarray:
    """blksprs/layouting/causal.py:124-142: the blocks of the compact mask are the active blocks that lie on
    the diagonal, at block offset ceil((window_size - 1) / block size) (windowed only), or in the block row
    of a partial last query block.  (The reference keeps no other block, also not the block one offset
    nearer that a window with (window_size - 1) % block size != 0 cuts as well.)  Plain loops."""
    s = sparsity_block_size
    lay = np.asarray(attention_layout) != 0
    out = np.zeros_like(lay)
    for b, length in enumerate(int(v) for v in valid_lengths):
        last = (length + s - 1) // s - 1
        for q in range(lay.shape[1]):
            for k in range(lay.shape[2]):
                keep = q == k
                if window_size is not None and q - k == (window_size - 1 + s - 1) // s:
                    keep = True
                if length % s != 0 and q == last and k <= last:
                    keep = True
                out[b, q, k] = keep and lay[b, q, k]
    return out


def contraction_lists(layout_x, layout_y, layout_o):
    """The work list implied by the reference kernel's scan (blksprs/ops/matmul.py:191-226): for every
    active output block, in row-major order, the ``(packed x index, packed y index)`` of every k where both
    operand blocks are active, ascending k.  Returns ``(pair_offsets int32 [nnz_o + 1], pairs int32 [T, 2])``.
    """
    lx, ly, lo = (np.asarray(a) != 0 for a in (layout_x, layout_y, layout_o))
    px = packed_indices(lx).reshape(lx.shape)
    py = packed_indices(ly).reshape(ly.shape)
    offsets, pairs = [0], []
    for b, i, j in np.argwhere(lo):
        ks = np.nonzero(lx[b, i, :] & ly[b, :, j])[0]
        pairs.extend((px[b, i, k], py[b, k, j]) for k in ks)
        offsets.append(len(pairs))
    return (np.asarray(offsets, dtype=np.int32),
            np.asarray(pairs, dtype=np.int32).reshape(-1, 2))


# --------------------------------------------------------------------------- conversion (bit exact)

def transpose(x, layout, sparsity_block_size: int):
    """blksprs/ops/transpose.py:13-52 (element transposition of every block, then flow_pull,
    blksprs/ops/flow.py:11-111): the compressed form of the transposed dense tensor under the transposed
    layout.  Returns ``(blocks in nonzero order of layout^T, layout^T)``."""
    lay = np.asarray(layout) != 0
    lay_t = np.ascontiguousarray(np.swapaxes(lay, -1, -2))
    px = packed_indices(lay).reshape(lay.shape)
    x = torch.as_tensor(x)
    out = [x[px[b, c, r]].transpose(-1, -2) for b, r, c in np.argwhere(lay_t)]
    s = sparsity_block_size
    res = torch.stack(out) if out else torch.empty((0, s, s), dtype=x.dtype)
    return res.contiguous(), lay_t



def to_sparse(x: torch.Tensor, layout, sbs: int) -> torch.Tensor:
    """blksprs/ops/conversion.py:230-276: the active ``sbs x sbs`` tiles of dense ``(B, R*sbs, C*sbs)`` in
    row-major block order (the reshape/permute identity of :127-138)."""
    lay = torch.as_tensor(np.asarray(layout) != 0)
    B, R, C = lay.shape
    tiles = x.reshape(B, R, sbs, C, sbs).permute(0, 1, 3, 2, 4)
    return tiles[lay].reshape(-1, sbs, sbs).clone()


def to_dense(x: torch.Tensor, layout, sbs: int, fill_value=0) -> torch.Tensor:
    """blksprs/ops/conversion.py:463-557: blocks scattered into a dense array pre-filled with ``fill_value``."""
    lay = torch.as_tensor(np.asarray(layout) != 0)
    B, R, C = lay.shape
    tiles = torch.full((B, R, C, sbs, sbs), fill_value, dtype=x.dtype)
    tiles[lay] = x
    return tiles.permute(0, 1, 3, 2, 4).reshape(B, R * sbs, C * sbs).clone()


# --------------------------------------------------------------------------- floating-point operators


def matmul(x, layout_x, y, layout_y, layout_o, sbs: int, acc_dtype=torch.float32) -> torch.Tensor:
    """blksprs/ops/matmul.py:186-253 via the recipe of test/cases/test_blocksparse.py:479-492:
    ``to_sparse(to_dense(x) @ to_dense(y), layout_o)`` accumulated in ``acc_dtype``, rounded to the input dtype."""
    xd = to_dense(x, layout_x, sbs).to(acc_dtype)
    yd = to_dense(y, layout_y, sbs).to(acc_dtype)
    return to_sparse(torch.matmul(xd, yd), layout_o, sbs).to(x.dtype)


def row_wise_reduce(x, layout, sbs: int, op: str, slice_only: bool = False):
    """blksprs/ops/misc/row_wise.py:103-205 (``op="sum"``) and :283-419 (``op="max"``): every block folds the
    reduction of each of its element rows into column 0 of the output block of its block row; the other
    columns keep the initial value (0 for the sum, ``-inf`` for the maximum); a row that holds a NaN gives NaN
    (:349-350); accumulation is wider than the storage type and the result is rounded once (:108-114, :146).
    Returns ``(values, (B, R, 1) layout)`` with values ``(rows, sbs, sbs)`` or ``(rows, sbs, 1)``."""
    lay = np.asarray(layout) != 0
    B, R, _ = lay.shape
    row_lay = lay.any(axis=-1, keepdims=True)
    row_index = packed_indices(row_lay)
    n_out = int(row_lay.sum())
    x = torch.as_tensor(x)
    start = 0.0 if op == "sum" else float("-inf")
    acc = torch.full((n_out, sbs, 1 if slice_only else sbs), start, dtype=torch.float64)
    for n, (b, r, _c) in enumerate(layout_indices(lay)):
        k = int(row_index[b * R + r])
        blk = x[n].to(torch.float64)
        if op == "sum":
            acc[k, :, 0] += blk.sum(dim=-1)
        else:
            acc[k, :, 0] = torch.maximum(acc[k, :, 0], blk.max(dim=-1).values)  # both propagate NaN
    return acc.to(x.dtype), row_lay


def row_wise_add(x, layout, y, sbs: int) -> torch.Tensor:
    """blksprs/ops/misc/row_wise.py:488-603: block ``(b, r, c)`` of x plus column 0 of the block of y that
    belongs to block row ``(b, r)``, broadcast over the columns; y holds ``sbs`` or 1 columns."""
    lay = np.asarray(layout) != 0
    B, R, _ = lay.shape
    row_index = packed_indices(lay.any(axis=-1, keepdims=True))
    x, y = torch.as_tensor(x), torch.as_tensor(y)
    out = torch.zeros_like(x)
    for n, (b, r, _c) in enumerate(layout_indices(lay)):
        k = int(row_index[b * R + r])
        out[n] = (x[n].to(torch.float64) + y[k, :, :1].to(torch.float64)).to(x.dtype)
    return out


def linear(x, layout, weight, bias, sbs: int):
    """blksprs/utils/processing.py:27-86: ``x @ weight^T (+ bias)`` on the dense form of x.  With a bias every
    output block is active (:57-62); without one, the block rows of x that hold a block, over all output columns
    (:63-64 with an all-ones weight layout).  Returns ``(blocks, layout)``."""
    lay = np.asarray(layout) != 0
    B, R, _ = lay.shape
    n_out = weight.shape[0] // sbs
    dense = to_dense(torch.as_tensor(x).to(torch.float64), lay, sbs)
    out = torch.nn.functional.linear(dense, weight.to(torch.float64), None if bias is None else bias.to(torch.float64))
    if bias is not None:
        lay_out = np.ones((B, R, n_out), dtype=bool)
    else:
        lay_out = np.broadcast_to(lay.any(axis=-1, keepdims=True), (B, R, n_out)).copy()
    return to_sparse(out, lay_out, sbs), lay_out


def softmax(x, layout, sbs: int) -> torch.Tensor:
    """blksprs/ops/softmax.py:524-570: per element row, softmax over the concatenation of the row's active
    blocks; inactive blocks act as ``-inf`` and rows without blocks do not exist in the output."""
    dense = to_dense(x.to(torch.float64), layout, sbs, fill_value=float("-inf"))
    lay = torch.as_tensor(np.asarray(layout) != 0)
    row_has_block = lay.any(dim=-1).repeat_interleave(sbs, dim=1)  # (B, R*sbs)
    out = torch.softmax(dense, dim=-1)
    out = torch.where(row_has_block.unsqueeze(-1), out, torch.zeros_like(out))
    return to_sparse(out, layout, sbs).to(x.dtype)


def softmax_backward(grad_out, y, layout, sbs: int) -> torch.Tensor:
    """blksprs/ops/softmax.py:581-638: ``dx = y * (g - sum_row(y * g))``."""
    yd = to_dense(y.to(torch.float64), layout, sbs)
    gd = to_dense(grad_out.to(torch.float64), layout, sbs)
    s = (yd * gd).sum(dim=-1, keepdim=True)
    return to_sparse(yd * (gd - s), layout, sbs).to(y.dtype)


def attention_scores_mask(attention_layout, sbs: int, mask=None, layout_mask=None, causal_lengths=None):
    """Boolean ``(B, Sq, Sk)`` array of ignored positions: outside the block layout
    (blksprs/ops/flash_attention.py:1049-1057), native causal predicate (:1128-1142), explicit mask where a
    mask block exists (:1146-1155)."""
    lay = torch.as_tensor(np.asarray(attention_layout) != 0)
    B, nq, nk = lay.shape
    ignored = ~lay.repeat_interleave(sbs, dim=1).repeat_interleave(sbs, dim=2)
    if causal_lengths is not None:
        qpos = torch.arange(nq * sbs).view(1, -1, 1)
        kpos = torch.arange(nk * sbs).view(1, 1, -1)
        length = torch.as_tensor(causal_lengths).view(-1, 1, 1)
        ignored = ignored | (kpos > qpos) | (qpos >= length) | (kpos >= length)
    if mask is not None:
        md = to_dense((mask != 0), layout_mask, sbs, fill_value=False)
        ignored = ignored | md
    return ignored


def flash_attention(q, layout_q, k, layout_k, v, layout_v, attention_layout, sbs: int, scale=None,
                    mask=None, layout_mask=None, bias=None, layout_bias=None, layout_o=None,
                    causal_lengths=None, acc_dtype=torch.float32):
    """blksprs/ops/flash_attention.py:1056-1224 restated densely, following the recipe of
    test/cases/test_blocksparse.py:1796-1828: ``scale * q k^T`` -> ``+ bias`` -> causal / layout / mask to
    ``-inf`` -> softmax -> NaN rows (nothing attended) to 0 -> ``@ v`` -> output layout.

    Inactive q/k head slices contribute zeros to the scores (:1074), inactive v slices contribute nothing,
    output slices inactive in ``layout_o`` are dropped.  Differentiable w.r.t. q, k, v, bias.
    Returns the compressed output (in ``q.dtype``).
    """
    qd = to_dense_autograd(q, layout_q, sbs).to(acc_dtype)
    kd = to_dense_autograd(k, layout_k, sbs).to(acc_dtype)
    vd = to_dense_autograd(v, layout_v, sbs).to(acc_dtype)
    head_dim = qd.shape[-1]
    if scale is None:
        scale = 1.0 if head_dim == 0 else 1.0 / math.sqrt(head_dim)
    scores = torch.matmul(qd, kd.transpose(-1, -2)) * scale
    if bias is not None:
        scores = scores + to_dense_autograd(bias, layout_bias, sbs).to(acc_dtype)
    ignored = attention_scores_mask(attention_layout, sbs, mask, layout_mask, causal_lengths)
    scores = scores.masked_fill(ignored, float("-inf"))
    all_ignored = ignored.all(dim=-1, keepdim=True)
    probs = torch.softmax(scores, dim=-1)
    probs = torch.where(all_ignored, torch.zeros_like(probs), probs)
    out = torch.matmul(probs, vd)
    if layout_o is None:
        layout_o = layout_matmul(attention_layout, layout_v)
    return to_sparse_autograd(out, layout_o, sbs).to(q.dtype)


def to_dense_autograd(x, layout, sbs: int):
    """``to_dense`` built from differentiable indexing (zeros outside the layout)."""
    lay = torch.as_tensor(np.asarray(layout) != 0)
    B, R, C = lay.shape
    tiles = torch.zeros((B, R, C, sbs, sbs), dtype=x.dtype)
    tiles = tiles.masked_scatter(lay.view(B, R, C, 1, 1).expand_as(tiles), x)
    return tiles.permute(0, 1, 3, 2, 4).reshape(B, R * sbs, C * sbs)


def to_sparse_autograd(x, layout, sbs: int):
    lay = torch.as_tensor(np.asarray(layout) != 0)
    B, R, C = lay.shape
    return x.reshape(B, R, sbs, C, sbs).permute(0, 1, 3, 2, 4)[lay].reshape(-1, sbs, sbs)


# --------------------------------------------------------------------------- seeded workloads


def random_layout(shape, density: float, generator: torch.Generator, ensure_rows: bool = False) -> torch.Tensor:
    """Bernoulli(density) block layout; with ``ensure_rows`` every row gets at least one block."""
    lay = torch.rand(shape, generator=generator) < density
    if ensure_rows and lay.numel():
        B, R, C = shape
        empty = ~lay.any(dim=-1)
        cols = torch.randint(0, C, (B, R), generator=generator)
        lay[empty, cols[empty]] = True
    return lay


def bigbird_layout(batch: int, n: int, generator: torch.Generator, window: int = 4, n_global: int = 2,
                   n_random: int = 3) -> torch.Tensor:
    """BigBird-style block layout: |i - j| <= window, the first ``n_global`` rows and columns, and
    ``n_random`` random columns per row."""
    i = torch.arange(n).view(-1, 1)
    j = torch.arange(n).view(1, -1)
    base = ((i - j).abs() <= window) | (j < n_global) | (i < n_global)
    lay = base.unsqueeze(0).repeat(batch, 1, 1)
    rnd = torch.rand((batch, n, n), generator=generator).argsort(dim=-1)[..., :n_random]
    lay.scatter_(2, rnd, True)
    return lay
