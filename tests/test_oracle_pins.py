"""Pins the CPU oracle: every oracle function is checked here against something that is not the
oracle's own formula - brute-force loops on tiny inputs, closed forms, torch library routines, and the
known answers the reference's own tests hold (test/cases/test_regressions.py, test_blocksparse.py).
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import blksprs_oracle as orc


def _layouts():
    g = torch.Generator().manual_seed(7)
    yield torch.zeros((1, 1, 1), dtype=torch.bool)
    yield torch.ones((1, 1, 1), dtype=torch.bool)
    yield torch.zeros((2, 3, 4), dtype=torch.bool)
    yield torch.ones((2, 3, 4), dtype=torch.bool)
    for shape, p in (((1, 4, 4), 0.5), ((3, 5, 7), 0.3), ((2, 8, 8), 0.8), ((4, 1, 9), 0.5)):
        yield torch.rand(shape, generator=g) < p


@pytest.mark.parametrize("layout", list(_layouts()))
def test_packed_indices_bruteforce(layout):
    flat = layout.reshape(-1).tolist()
    expected, seen = [], 0
    for v in flat:
        expected.append(seen if v else -1)
        seen += int(v)
    got = orc.packed_indices(layout.numpy())
    assert got.dtype == np.int64 and got.tolist() == expected


@pytest.mark.parametrize("layout", list(_layouts()))
def test_layout_indices_is_torch_nonzero(layout):
    assert np.array_equal(orc.layout_indices(layout.numpy()), torch.nonzero(layout).numpy())
    assert orc.n_sparse_blocks(layout.numpy()) == int(layout.sum())


def test_block_count_is_exact_for_half_precision_layouts():
    # test_regressions.py:1060-1075: 65536 ones in an fp16 layout must count exactly
    layout = torch.ones((1, 256, 256), dtype=torch.float16)
    assert orc.n_sparse_blocks(layout.numpy()) == 65536


@pytest.mark.parametrize("layout", list(_layouts()))
def test_segmented_indices_bruteforce(layout):
    B, R, C = layout.shape
    indices, offsets, longest = orc.segmented_indices(layout.numpy())
    exp_idx, exp_off, exp_long = [], [0], 0
    for b in range(B):
        for r in range(R):
            cols = [c for c in range(C) if layout[b, r, c]]
            exp_idx += cols
            exp_off.append(len(exp_idx))
            exp_long = max(exp_long, len(cols))
    if exp_long == 0:
        # flash_attention.py:1928-1938: (empty, zeros, 1)
        assert indices.size == 0 and offsets.tolist() == [0] * (B * R + 1) and longest == 1
    else:
        assert indices.tolist() == exp_idx and offsets.tolist() == exp_off and longest == exp_long
    assert indices.dtype == np.int32 and offsets.dtype == np.int32


def test_segmented_index_dtype_truth_table():
    # test_regressions.py:1037-1047
    assert orc.segmented_index_dtype(0, 1) == np.int32
    assert orc.segmented_index_dtype(2_147_483_647, 2_147_483_648) == np.int32
    assert orc.segmented_index_dtype(2_147_483_648, 1) == np.int64
    assert orc.segmented_index_dtype(1, 2_147_483_649) == np.int64


@pytest.mark.parametrize("layout", list(_layouts()))
def test_sorted_packed_indices_against_torch_sort(layout):
    packed = torch.from_numpy(orc.packed_indices(layout.numpy())).reshape(layout.shape)
    expected = packed.sort(descending=True, dim=-1)[0].reshape(-1)
    got, mbl = orc.sorted_packed_indices(layout.numpy())
    assert np.array_equal(got, expected.numpy())
    longest = int(layout.sum(dim=-1).max()) if layout.numel() else 0
    assert mbl == max(2, 1 << max(longest - 1, 0).bit_length()) and mbl >= longest and (mbl & (mbl - 1)) == 0


def test_layout_matmul_bruteforce_and_float_bmm():
    g = torch.Generator().manual_seed(3)
    lx = torch.rand((3, 5, 6), generator=g) < 0.3
    ly = torch.rand((3, 6, 4), generator=g) < 0.3
    got = orc.layout_matmul(lx.numpy(), ly.numpy())
    brute = np.zeros((3, 5, 4), dtype=bool)
    for b in range(3):
        for i in range(5):
            for j in range(4):
                brute[b, i, j] = any(lx[b, i, k] and ly[b, k, j] for k in range(6))
    assert np.array_equal(got, brute)
    assert np.array_equal(got, torch.matmul(lx.float(), ly.float()).bool().numpy())
    # empty inner dimension: nothing is active (test_regressions.py:1208-1217)
    assert not orc.layout_matmul(np.ones((1, 2, 0)), np.ones((1, 0, 3))).any()


def test_build_sparsity_layout_bruteforce_and_known_answers():
    """Loops over blocks and elements on tiny inputs; the reference's own facts (NaN activates a block:
    test/cases/test_regressions.py:1943-1980; a to_dense round trip gives back the layout:
    test/cases/test_blocksparse.py:990-1009); -0.0 equals 0 in IEEE comparison."""
    g = torch.Generator().manual_seed(5)
    s = 4
    x = torch.randn((2, 3 * s, 5 * s), generator=g)
    keep = torch.rand((2, 3, 5), generator=g) < 0.4
    x = x * keep.repeat_interleave(s, 1).repeat_interleave(s, 2)
    x[0, 0, 0] = -0.0 if not keep[0, 0, 0] else x[0, 0, 0]
    brute = np.zeros((2, 3, 5), dtype=bool)
    for b in range(2):
        for r in range(3):
            for c in range(5):
                for i in range(s):
                    for j in range(s):
                        if x[b, r * s + i, c * s + j].item() != 0:
                            brute[b, r, c] = True
    got = orc.build_sparsity_layout(x, s)
    assert np.array_equal(got, brute)
    assert np.array_equal(got, keep.numpy())  # random normal values are never exactly zero
    for dtype in (torch.float16, torch.bfloat16, torch.float32, torch.float64):
        d = torch.zeros((1, s, 2 * s), dtype=dtype)
        d[0, 0, s] = float("nan")
        assert np.array_equal(orc.build_sparsity_layout(d, s), np.array([[[False, True]]]))
        d[0, 0, s] = -0.0
        assert not orc.build_sparsity_layout(d, s).any()
    ints = torch.zeros((1, s, s), dtype=torch.int32)
    ints[0, 3, 3] = -1
    assert orc.build_sparsity_layout(ints, s).all()


def test_contraction_lists_reproduce_the_dense_product():
    """The lists are a regrouping of a block matmul: summing x[px] @ y[py] per output block must equal the
    dense masked product; and within a block k ascends."""
    g = torch.Generator().manual_seed(11)
    sbs = 4
    lx = torch.rand((2, 3, 5), generator=g) < 0.5
    ly = torch.rand((2, 5, 4), generator=g) < 0.5
    lo = torch.rand((2, 3, 4), generator=g) < 0.7  # includes blocks with no contributing k
    x = torch.randn((int(lx.sum()), sbs, sbs), generator=g, dtype=torch.float64)
    y = torch.randn((int(ly.sum()), sbs, sbs), generator=g, dtype=torch.float64)
    offsets, pairs = orc.contraction_lists(lx.numpy(), ly.numpy(), lo.numpy())
    n_o = int(lo.sum())
    assert offsets.shape == (n_o + 1,) and offsets[0] == 0 and offsets[-1] == len(pairs)
    out = torch.zeros((n_o, sbs, sbs), dtype=torch.float64)
    for n in range(n_o):
        seg = pairs[offsets[n]:offsets[n + 1]]
        assert np.all(np.diff(seg[:, 0]) > 0)  # x blocks of one row are stored in ascending k
        for px, py in seg:
            out[n] += x[px] @ y[py]
    dense = orc.to_dense(x, lx.numpy(), sbs) @ orc.to_dense(y, ly.numpy(), sbs)
    assert torch.allclose(out, orc.to_sparse(dense, lo.numpy(), sbs), atol=1e-12)
    total = int(np.einsum("bik,bkj,bij->", lx.numpy().astype(int), ly.numpy().astype(int), lo.numpy().astype(int)))
    assert len(pairs) == total


def test_conversion_against_slice_loops():
    # the loop form of test_blocksparse.py:1674-1699
    g = torch.Generator().manual_seed(5)
    sbs = 4
    layout = torch.rand((2, 3, 5), generator=g) < 0.5
    x = torch.randn((2, 3 * sbs, 5 * sbs), generator=g)
    blocks = orc.to_sparse(x, layout.numpy(), sbs)
    dense = orc.to_dense(blocks, layout.numpy(), sbs, fill_value=7.5)
    n = 0
    for b in range(2):
        for r in range(3):
            for c in range(5):
                tile = x[b, r * sbs:(r + 1) * sbs, c * sbs:(c + 1) * sbs]
                got = dense[b, r * sbs:(r + 1) * sbs, c * sbs:(c + 1) * sbs]
                if layout[b, r, c]:
                    assert torch.equal(blocks[n], tile) and torch.equal(got, tile)
                    n += 1
                else:
                    assert torch.all(got == 7.5)
    assert n == blocks.size(0)


def test_transpose_is_the_conversion_of_the_transposed_dense_tensor():
    """transpose(to_sparse(d, l), l) == to_sparse(d^T, l^T) for every dense d (the defining property, checked
    through the independently pinned conversion), twice is the identity, and the layout returned is l^T."""
    g = torch.Generator().manual_seed(11)
    s = 4
    layout = (torch.rand((3, 2, 5), generator=g) < 0.5).numpy()
    dense = torch.randn((3, 2 * s, 5 * s), generator=g)
    blocks = orc.to_sparse(dense, layout, s)
    got, layout_t = orc.transpose(blocks, layout, s)
    assert np.array_equal(layout_t, np.swapaxes(layout, 1, 2))
    assert torch.equal(got, orc.to_sparse(dense.transpose(1, 2).contiguous(), layout_t, s))
    back, layout_tt = orc.transpose(got, layout_t, s)
    assert np.array_equal(layout_tt, layout) and torch.equal(back, blocks)
    empty, _ = orc.transpose(torch.empty((0, s, s)), np.zeros((1, 2, 3), bool), s)
    assert empty.shape == (0, s, s)


def test_row_wise_reductions_against_dense_torch_and_loops():
    """sum / max of the dense tensor (inactive blocks filled with the neutral element) for every row that holds
    a block; element-by-element loops on the same input; columns other than 0 keep the neutral element; the
    reference's own facts: NaN wins over everything in the maximum, also from a second block
    (test/cases/test_regressions.py:1981-2004), a row of -inf stays -inf (:1173-1183)."""
    g = torch.Generator().manual_seed(21)
    s = 4
    layout = (torch.rand((2, 3, 5), generator=g) < 0.5).numpy()
    layout[1, 2, :] = False  # a block row without blocks
    dense = torch.randn((2, 3 * s, 5 * s), generator=g, dtype=torch.float64)
    blocks = orc.to_sparse(dense, layout, s)
    rows = layout.any(-1)
    for op, neutral, ref in (("sum", 0.0, lambda d: d.sum(-1)), ("max", float("-inf"), lambda d: d.max(-1).values)):
        filled = orc.to_dense(blocks, layout, s, fill_value=neutral)
        out, row_layout = orc.row_wise_reduce(blocks, layout, s, op)
        assert row_layout.shape == (2, 3, 1) and np.array_equal(row_layout[..., 0], rows)
        assert out.shape == (int(rows.sum()), s, s)
        got = orc.to_dense(out, row_layout, s, fill_value=neutral)  # (B, R*s, s)
        expected = ref(filled)
        row_mask = torch.as_tensor(rows).repeat_interleave(s, 1)
        assert torch.allclose(got[..., 0][row_mask], expected[row_mask], atol=1e-12)
        assert torch.all(out[..., 1:] == neutral)
        sliced, _ = orc.row_wise_reduce(blocks, layout, s, op, slice_only=True)
        assert sliced.shape == (int(rows.sum()), s, 1) and torch.equal(sliced[..., 0], out[..., 0])
        # loops
        k = 0
        for b in range(2):
            for r in range(3):
                if not rows[b, r]:
                    continue
                for e in range(s):
                    vals = [dense[b, r * s + e, c * s + j].item() for c in range(5) if layout[b, r, c] for j in range(s)]
                    want = sum(vals) if op == "sum" else max(vals)
                    assert abs(out[k, e, 0].item() - want) < 1e-12
                k += 1
    two = np.ones((1, 1, 2), dtype=bool)
    d = torch.arange(2.0 * s * s).reshape(1, s, 2 * s)
    d[0, 0, 0] = float("nan")
    d[0, 1, s] = float("nan")
    d[0, 2, :] = float("-inf")
    out, _ = orc.row_wise_reduce(orc.to_sparse(d, two, s), two, s, "max", slice_only=True)
    assert torch.isnan(out[0, 0, 0]) and torch.isnan(out[0, 1, 0]) and torch.isneginf(out[0, 2, 0])
    assert out[0, 3, 0] == d[0, 3].max()


def test_row_wise_add_is_a_broadcast_add_on_the_dense_tensor():
    """to_dense(row_wise_add(x, y)) == (dense + row values) on active blocks and 0 elsewhere, for slices and for
    square blocks of y (only column 0 counts); adding the negated row sum of a one-block row centres it."""
    g = torch.Generator().manual_seed(22)
    s = 4
    layout = (torch.rand((2, 3, 4), generator=g) < 0.6).numpy()
    layout[0, 1, :] = False
    dense = torch.randn((2, 3 * s, 4 * s), generator=g, dtype=torch.float64)
    blocks = orc.to_sparse(dense, layout, s)
    rows = layout.any(-1)
    n_rows = int(rows.sum())
    y = torch.randn((n_rows, s, 1), generator=g, dtype=torch.float64)
    y_dense = torch.zeros((2, 3, s), dtype=torch.float64)
    y_dense[torch.as_tensor(rows)] = y[..., 0]
    expected = orc.to_dense(orc.to_sparse(dense + y_dense.reshape(2, 3 * s, 1), layout, s), layout, s)
    got = orc.row_wise_add(blocks, layout, y, s)
    assert torch.allclose(orc.to_dense(got, layout, s), expected, atol=1e-12)
    y_square = torch.randn((n_rows, s, s), generator=g, dtype=torch.float64)
    y_square[..., 0] = y[..., 0]
    assert torch.equal(orc.row_wise_add(blocks, layout, y_square, s), got)
    one = np.ones((1, 1, 1), dtype=bool)
    blk = torch.randn((1, s, s), generator=g, dtype=torch.float64)
    total, _ = orc.row_wise_reduce(blk, one, s, "sum", slice_only=True)
    centred = orc.row_wise_add(blk, one, -total / s, s)
    assert torch.allclose(centred.sum(-1), torch.zeros((1, s), dtype=torch.float64), atol=1e-12)


def test_linear_is_the_block_matmul_with_the_replicated_weight_plus_bias():
    """The reference's own construction (blksprs/utils/processing.py:48-83): a block matmul with the transposed
    weight repeated over the batch under an all-ones layout, then the bias added to every row, through the
    independently pinned matmul; and a loop over output elements on a tiny case."""
    g = torch.Generator().manual_seed(31)
    s = 4
    layout = (torch.rand((2, 3, 2), generator=g) < 0.6).numpy()
    layout[1, 0, :] = False
    x = orc.to_sparse(torch.randn((2, 3 * s, 2 * s), generator=g, dtype=torch.float64), layout, s)
    weight = torch.randn((3 * s, 2 * s), generator=g, dtype=torch.float64)
    bias = torch.randn((3 * s,), generator=g, dtype=torch.float64)
    layout_w = np.ones((2, 2, 3), dtype=bool)
    w_blocks = orc.to_sparse(weight.t().unsqueeze(0).repeat(2, 1, 1).contiguous(), layout_w, s)
    dense_x = orc.to_dense(x, layout, s)
    for b in (None, bias):
        got, lay_out = orc.linear(x, layout, weight, b, s)
        product = orc.matmul(x, layout, w_blocks, layout_w, lay_out, s, acc_dtype=torch.float64)
        want = orc.to_dense(product, lay_out, s)
        if b is not None:
            want = want + b
            assert lay_out.all()
        else:
            assert np.array_equal(lay_out[..., 0], layout.any(-1)) and (lay_out == lay_out[..., :1]).all()
        assert torch.allclose(orc.to_dense(got, lay_out, s), orc.to_dense(orc.to_sparse(want, lay_out, s), lay_out, s),
                              atol=1e-12)
    got, lay_out = orc.linear(x, layout, weight, bias, s)
    dense_out = orc.to_dense(got, lay_out, s)
    for bi, i, j in ((0, 0, 0), (1, 2, 5), (1, 11, 11), (0, 7, 3)):
        want = sum(dense_x[bi, i, k].item() * weight[j, k].item() for k in range(2 * s)) + bias[j].item()
        assert abs(dense_out[bi, i, j].item() - want) < 1e-12


def test_matmul_full_layout_is_bmm_and_inactive_blocks_do_not_contribute():
    g = torch.Generator().manual_seed(2)
    sbs = 4
    full = np.ones((2, 2, 2), dtype=bool)
    a = torch.randn((2, 8, 8), generator=g, dtype=torch.float64)
    b = torch.randn((2, 8, 8), generator=g, dtype=torch.float64)
    out = orc.matmul(orc.to_sparse(a, full, sbs), full, orc.to_sparse(b, full, sbs), full, full, sbs,
                     acc_dtype=torch.float64)
    assert torch.allclose(orc.to_dense(out, full, sbs), torch.bmm(a, b), atol=1e-12)
    # x with only block (0,0): output row 0 equals a00 @ b0*, row 1 is zero
    lx = np.zeros((1, 2, 2), dtype=bool)
    lx[0, 0, 0] = True
    one = np.ones((1, 2, 2), dtype=bool)
    out = orc.matmul(a[:1, :4, :4].clone(), lx, orc.to_sparse(b[:1], one, sbs), one, one, sbs,
                     acc_dtype=torch.float64)
    dense = orc.to_dense(out, one, sbs)
    assert torch.allclose(dense[0, :4], a[0, :4, :4] @ b[0, :4, :], atol=1e-12)
    assert torch.all(dense[0, 4:] == 0)


def test_softmax_matches_per_row_softmax_over_concatenated_blocks():
    g = torch.Generator().manual_seed(9)
    sbs = 4
    layout = torch.rand((2, 3, 4), generator=g) < 0.5
    layout[0, 1] = False  # a row without blocks
    x = torch.randn((int(layout.sum()), sbs, sbs), generator=g)
    out = orc.softmax(x, layout.numpy(), sbs)
    lidx = torch.nonzero(layout)
    for b in range(2):
        for r in range(3):
            ids = [n for n, (bb, rr, _) in enumerate(lidx.tolist()) if bb == b and rr == r]
            if not ids:
                continue
            for e in range(sbs):
                row = torch.cat([x[n, e] for n in ids]).double()
                expected = torch.softmax(row, dim=0)
                got = torch.cat([out[n, e] for n in ids]).double()
                assert torch.allclose(got, expected, atol=1e-6)
    # backward formula against autograd
    y = out.double().requires_grad_(False)
    grad = torch.randn(x.shape, generator=g).double()
    xd = orc.to_dense(x.double(), layout.numpy(), sbs, fill_value=float("-inf")).requires_grad_(True)
    sm = torch.softmax(xd, dim=-1)
    sm = torch.nan_to_num(sm, nan=0.0)
    (sm * orc.to_dense(grad, layout.numpy(), sbs)).sum().backward()
    expected = orc.to_sparse(torch.nan_to_num(xd.grad, nan=0.0), layout.numpy(), sbs)
    assert torch.allclose(orc.softmax_backward(grad, y, layout.numpy(), sbs), expected, atol=1e-9)


def _full(b, r, c):
    return np.ones((b, r, c), dtype=bool)


def test_attention_full_layout_is_sdpa():
    # test_regressions.py:488-527: full layout without mask equals scaled_dot_product_attention
    g = torch.Generator().manual_seed(4)
    sbs, B, S, D = 4, 2, 8, 8
    q, k, v = (torch.randn((B, S, D), generator=g, dtype=torch.float64) for _ in range(3))
    lq = _full(B, S // sbs, D // sbs)
    la = _full(B, S // sbs, S // sbs)
    out = orc.flash_attention(orc.to_sparse(q, lq, sbs), lq, orc.to_sparse(k, lq, sbs), lq,
                              orc.to_sparse(v, lq, sbs), lq, la, sbs, acc_dtype=torch.float64)
    assert torch.allclose(orc.to_dense(out, lq, sbs), F.scaled_dot_product_attention(q, k, v), atol=1e-12)
    # causal lengths equal an explicit is_causal mask when the length covers the sequence
    out = orc.flash_attention(orc.to_sparse(q, lq, sbs), lq, orc.to_sparse(k, lq, sbs), lq,
                              orc.to_sparse(v, lq, sbs), lq, la, sbs, causal_lengths=torch.full((B,), S),
                              acc_dtype=torch.float64)
    assert torch.allclose(orc.to_dense(out, lq, sbs), F.scaled_dot_product_attention(q, k, v, is_causal=True),
                          atol=1e-12)


def test_attention_known_answers_from_reference_tests():
    sbs = 4
    # uniform attention (test_regressions.py:63-94): q = k = 0, v = 1 -> output exactly 1
    lq = _full(1, 1, 1)
    lk = _full(1, 8, 1)
    la = _full(1, 1, 8)
    out = orc.flash_attention(torch.zeros((1, sbs, sbs)), lq, torch.zeros((8, sbs, sbs)), lk,
                              torch.ones((8, sbs, sbs)), lk, la, sbs)
    assert torch.all(out == 1)
    # uniform gradient (test_regressions.py:97-129): many queries, one key block -> dV = n_query / n_key
    lq = _full(1, 5, 1)
    lk = _full(1, 1, 1)
    la = _full(1, 5, 1)
    v = torch.ones((1, sbs, sbs), requires_grad=True)
    out = orc.flash_attention(torch.zeros((5, sbs, sbs)), lq, torch.zeros((1, sbs, sbs)), lk, v, lk, la, sbs)
    out.sum().backward()
    assert torch.all(v.grad == (5 * sbs) / sbs)
    # zero-width QK head dimension: scores are 0, scale defaults to 1 (test_regressions.py:1256-1283)
    lq0 = np.ones((1, 2, 0), dtype=bool)
    lv = _full(1, 2, 1)
    la = _full(1, 2, 2)
    vv = torch.randn((2, sbs, sbs))
    out = orc.flash_attention(torch.zeros((0, sbs, sbs)), lq0, torch.zeros((0, sbs, sbs)), lq0, vv, lv, la, sbs)
    mean = orc.to_dense(vv, lv, sbs).mean(dim=1, keepdim=True).expand(1, 2 * sbs, sbs)
    assert torch.allclose(orc.to_dense(out, lv, sbs), mean, atol=1e-6)


def test_attention_finite_bias_is_added_unscaled_before_the_softmax():
    """A finite additive bias against ``F.scaled_dot_product_attention(attn_mask=bias)``, which adds a float
    mask to the scaled scores: a bias multiplied by the scale, added after the softmax or subtracted would
    differ.  Gradients of q, k, v and the bias against torch's own."""
    g = torch.Generator().manual_seed(21)
    sbs, B, S, D = 4, 2, 12, 8
    lq, la = _full(B, S // sbs, D // sbs), _full(B, S // sbs, S // sbs)
    dense = [torch.randn((B, S, D), generator=g, dtype=torch.float64).requires_grad_(True) for _ in range(3)]
    bias = (3.0 * torch.randn((B, S, S), generator=g, dtype=torch.float64)).requires_grad_(True)
    sparse = [orc.to_sparse_autograd(t, lq, sbs) for t in dense]
    out = orc.flash_attention(sparse[0], lq, sparse[1], lq, sparse[2], lq, la, sbs, scale=0.3,
                              bias=orc.to_sparse_autograd(bias, la, sbs), layout_bias=la, acc_dtype=torch.float64)
    go = torch.randn((B, S, D), generator=g, dtype=torch.float64)
    got = torch.autograd.grad(orc.to_dense_autograd(out, lq, sbs), (*dense, bias), go)
    ref_in = [t.detach().clone().requires_grad_(True) for t in (*dense, bias)]
    ref = F.scaled_dot_product_attention(ref_in[0], ref_in[1], ref_in[2], attn_mask=ref_in[3], scale=0.3)
    assert torch.allclose(orc.to_dense(out.detach(), lq, sbs), ref.detach(), atol=1e-12)
    for a, b in zip(got, torch.autograd.grad(ref, ref_in, go)):
        assert torch.allclose(a, b, atol=1e-12)


def test_attention_mask_bias_order_and_fully_masked_rows():
    g = torch.Generator().manual_seed(8)
    sbs, S = 4, 8
    lq = _full(1, 2, 1)
    la = _full(1, 2, 2)
    q, k, v = (orc.to_sparse(torch.randn((1, S, sbs), generator=g), lq, sbs) for _ in range(3))
    # +inf bias under a mask stays ignored (test_regressions.py:2075-2120)
    bias = torch.zeros((1, S, S))
    bias[0, :, 0] = float("inf")
    mask = torch.zeros((1, S, S), dtype=torch.bool)
    mask[0, :, 0] = True
    mask[0, 3, :] = True  # one fully masked query row -> output 0, no NaN
    out = orc.flash_attention(q, lq, k, lq, v, lq, la, sbs, mask=orc.to_sparse(mask, la, sbs), layout_mask=la,
                              bias=orc.to_sparse(bias, la, sbs), layout_bias=la)
    dense = orc.to_dense(out, lq, sbs)
    assert torch.isfinite(dense).all() and torch.all(dense[0, 3] == 0)
    # brute force for one unmasked row
    qd, kd, vd = (orc.to_dense(t, lq, sbs)[0] for t in (q, k, v))
    s = (qd[1] @ kd.T) / math.sqrt(sbs)
    w = torch.softmax(s[1:], dim=0)
    assert torch.allclose(dense[0, 1], w @ vd[1:], atol=1e-6)
    # block layout: a query block that attends nothing yields zeros and the default output layout follows
    # attention (x) v (test_regressions.py:488-532)
    la2 = np.array([[[1, 0], [0, 0]]], dtype=bool)
    out = orc.flash_attention(q, lq, k, lq, v, lq, la2, sbs)
    assert out.shape[0] == 1
    w = torch.softmax((qd[:4] @ kd[:4].T) / math.sqrt(sbs), dim=-1)
    assert torch.allclose(out[0], w @ vd[:4], atol=1e-6)
