"""Writes the golden fixtures of this directory: small, fixed inputs together with the outputs the CPU oracle
gives for them.  The GPU parity tests and the oracle's own tests compare against these files, so a change of
either the kernels or the oracle that alters a result shows up as a diff of a committed file.

    python tests/golden/make_fixtures.py

The inputs are stored next to the outputs (nothing depends on a random number generator at test time).
Expected outputs of the integer functions are exact; floating-point outputs are float64.
"""

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))

from oracle import blksprs_oracle as orc  # noqa: E402


def lut_fixture():
    g = torch.Generator().manual_seed(11)
    lx = orc.random_layout((2, 5, 7), 0.45, g, ensure_rows=True).numpy()
    ly = orc.random_layout((2, 7, 6), 0.5, g, ensure_rows=True).numpy()
    lo = orc.layout_matmul(lx, ly)
    off, pairs = orc.contraction_lists(lx, ly, lo)
    csr_idx, csr_off, longest = orc.segmented_indices(lx)
    sorted_rows, max_blocks_line = orc.sorted_packed_indices(lx)
    np.savez(HERE / "lut.npz", layout_x=lx, layout_y=ly, layout_o=lo, packed_x=orc.packed_indices(lx),
             nonzero_o=orc.layout_indices(lo), pair_offsets=off, pairs=pairs, csr_indices=csr_idx,
             csr_offsets=csr_off, csr_longest=np.int64(longest), sorted_rows=sorted_rows,
             max_blocks_line=np.int64(max_blocks_line))


def compute_fixture():
    g = torch.Generator().manual_seed(12)
    sbs = 16
    lx = orc.random_layout((2, 3, 4), 0.6, g, ensure_rows=True)
    ly = orc.random_layout((2, 4, 3), 0.6, g, ensure_rows=True)
    lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
    x = torch.randn((int(lx.sum()), sbs, sbs), generator=g, dtype=torch.float64) / 8
    y = torch.randn((int(ly.sum()), sbs, sbs), generator=g, dtype=torch.float64)
    mm = orc.matmul(x, lx.numpy(), y, ly.numpy(), lo.numpy(), sbs, acc_dtype=torch.float64)
    sm = orc.softmax(x * 16, lx.numpy(), sbs)
    # attention: 2 batch entries, 3 query blocks, 4 key blocks, one head slice, mask on part of the layout
    la = orc.random_layout((2, 3, 4), 0.7, g, ensure_rows=True)
    full_q = torch.ones((2, 3, 1), dtype=torch.bool)
    full_k = torch.ones((2, 4, 1), dtype=torch.bool)
    q = torch.randn((6, sbs, sbs), generator=g, dtype=torch.float64)
    k = torch.randn((8, sbs, sbs), generator=g, dtype=torch.float64)
    v = torch.randn((8, sbs, sbs), generator=g, dtype=torch.float64)
    lmask = la & orc.random_layout((2, 3, 4), 0.6, g)
    mask = torch.rand((int(lmask.sum()), sbs, sbs), generator=g) < 0.3
    at = orc.flash_attention(q, full_q.numpy(), k, full_k.numpy(), v, full_k.numpy(), la.numpy(), sbs, mask=mask,
                             layout_mask=lmask.numpy(), acc_dtype=torch.float64)
    np.savez(HERE / "compute.npz", sbs=np.int64(sbs), layout_x=lx.numpy(), layout_y=ly.numpy(), layout_o=lo.numpy(),
             x=x.numpy(), y=y.numpy(), matmul=mm.numpy(), softmax_in=(x * 16).numpy(), softmax=sm.numpy(),
             attention_layout=la.numpy(), q=q.numpy(), k=k.numpy(), v=v.numpy(), layout_mask=lmask.numpy(),
             mask=mask.numpy(), attention=at.numpy())


def neighbours_fixture():
    """The operations next to the hot path: transpose, layout of a dense tensor, row-wise sum / max / add, a
    linear layer with bias, causal layouts and compact masks."""
    g = torch.Generator().manual_seed(13)
    sbs = 16
    layout = orc.random_layout((2, 3, 4), 0.6, g, ensure_rows=True).numpy()
    layout[1, 2, :] = False
    x = torch.randn((int(layout.sum()), sbs, sbs), generator=g, dtype=torch.float64)
    xt, layout_t = orc.transpose(x, layout, sbs)
    dense = orc.to_dense(x, layout, sbs)
    row_sum, row_layout = orc.row_wise_reduce(x, layout, sbs, "sum")
    row_max, _ = orc.row_wise_reduce(x, layout, sbs, "max", slice_only=True)
    centred = orc.row_wise_add(x, layout, -row_max, sbs)
    weight = torch.randn((2 * sbs, 4 * sbs), generator=g, dtype=torch.float64) / 8
    bias = torch.randn((2 * sbs,), generator=g, dtype=torch.float64)
    lin, lin_layout = orc.linear(x, layout, weight, bias, sbs)
    lengths = np.array([37, 64, 1], dtype=np.int64)
    causal = orc.causal_layout(lengths, sbs)
    window = orc.causal_layout(lengths, sbs, window_size=23)
    np.savez(HERE / "neighbours.npz", sbs=np.int64(sbs), layout=layout, x=x.numpy(), transposed=xt.numpy(),
             layout_t=layout_t, dense_layout=orc.build_sparsity_layout(dense, sbs), row_layout=row_layout,
             row_sum=row_sum.numpy(), row_max=row_max.numpy(), centred=centred.numpy(), weight=weight.numpy(),
             bias=bias.numpy(), linear=lin.numpy(), linear_layout=lin_layout, lengths=lengths, causal_layout=causal,
             window_layout=window, causal_mask_layout=orc.causal_mask_layout(lengths, causal, sbs),
             window_mask_layout=orc.causal_mask_layout(lengths, window, sbs, window_size=23))


if __name__ == "__main__":
    lut_fixture()
    compute_fixture()
    neighbours_fixture()
    print("wrote", sorted(p.name for p in HERE.glob("*.npz")))
