"""Parity of the block-sparse softmax (fp32, rtol = atol = 1e-5) with the CPU oracle."""

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import assert_close, rand_blocks, rand_layout

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [(16, (2, 3, 4), 0.5), (16, (1, 1, 40), 1.0), (32, (2, 4, 4), 0.6), (64, (2, 4, 8), 0.5),
         (64, (1, 2, 40), 1.0), (128, (1, 2, 3), 0.7), (256, (1, 1, 2), 1.0), (64, (2, 8, 8), 0.15)]


@pytest.mark.parametrize("sbs,shape,density", CASES)
@pytest.mark.parametrize("flag_fused", [True, False])
def test_forward_and_backward(device, sbs, shape, density, flag_fused):
    layout = rand_layout(shape, density, seed=sbs + shape[2])
    n = int(layout.sum())
    x = rand_blocks(n, sbs, torch.float32, seed=1, scale=2.0)
    xd = x.to(device).requires_grad_(True)
    out = bs.ops.softmax(xd, layout.to(device), sbs, flag_fused=flag_fused)
    assert isinstance(out, bs.BlksprsTensor) and out.dtype == torch.float32
    assert_close(out, orc.softmax(x, layout.numpy(), sbs), TOL, "softmax forward")
    g = rand_blocks(n, sbs, torch.float32, seed=2)
    out.backward(g.to(device))
    expected = orc.softmax_backward(g, orc.softmax(x, layout.numpy(), sbs), layout.numpy(), sbs)
    assert_close(xd.grad, expected, TOL, "softmax backward")


def test_rows_sum_to_one_at_config3_size(device):
    """Config 3 at full size (B=32, 2048x2048, sbs 64, causal + 10 %): every element row sums to 1, and three
    batch entries (first, middle, last) match the oracle, forward and backward; a second run gives the same bits."""
    B, n, sbs = 32, 32, 64
    g = torch.Generator().manual_seed(0)
    tri = torch.tril(torch.ones((n, n), dtype=torch.bool))
    layout = tri.unsqueeze(0) | ((torch.rand((B, n, n), generator=g) < 0.1) & ~tri)
    nnz = int(layout.sum())
    x = torch.randn((nnz, sbs, sbs), generator=g) * 2.0
    out = bs.ops.softmax(x.to(device), layout.to(device), sbs)
    dense = bs.ops.to_dense(out, layout.to(device), sbs)
    sums = dense.sum(dim=-1)
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-5)
    # forward and backward of the first, a middle and the last batch entry against the oracle
    starts = torch.cumsum(layout.reshape(B, -1).sum(dim=1), 0).tolist()
    gout = torch.randn((nnz, sbs, sbs), generator=g)
    xd = x.to(device).requires_grad_(True)
    od = bs.ops.softmax(xd, layout.to(device), sbs)
    assert torch.equal(od.detach(), out)
    od.backward(gout.to(device))
    for b in (0, B // 2, B - 1):
        lo, hi = (starts[b - 1] if b else 0), starts[b]
        lb = layout[b:b + 1].numpy()
        want = orc.softmax(x[lo:hi], lb, sbs)
        assert_close(out[lo:hi], want, TOL, f"batch {b}")
        assert_close(xd.grad[lo:hi], orc.softmax_backward(gout[lo:hi], want, lb, sbs), TOL, f"batch {b} backward")


def test_non_contiguous_gradient_and_extremes(device):
    # reference: test_regressions.py:192-208 (gradient views) and -inf / large logits
    sbs = 16
    layout = torch.ones((1, 1, 2), dtype=torch.bool)
    x = torch.randn((2, sbs, sbs))
    x[0, 0, :] = float("-inf")
    x[1, 0, :] = float("-inf")
    x[1, 0, 3] = 0.0
    x[0, 1, :] = 1e4
    xd = x.to(device).requires_grad_(True)
    out = bs.ops.softmax(xd, layout.to(device), sbs)
    exp = orc.softmax(x, layout.numpy(), sbs)
    assert_close(out, exp, TOL, "extreme logits")
    base = torch.randn((2, sbs, sbs * 2), device=device)
    grad = base[:, :, ::2]
    assert not grad.is_contiguous()
    out.backward(grad)
    expected = orc.softmax_backward(grad.cpu().contiguous(), exp, layout.numpy(), sbs)
    assert_close(xd.grad, expected, TOL, "non-contiguous grad")


@pytest.mark.parametrize("layout_shape", [(0, 1, 1), (1, 0, 1), (1, 1, 0)])
@pytest.mark.parametrize("flag_fused", [True, False])
def test_empty_layouts(device, layout_shape, flag_fused):
    # reference: test_regressions.py:1186-1197
    layout = torch.ones(layout_shape, dtype=torch.bool, device=device)
    x = torch.empty((0, 16, 16), device=device)
    out = bs.ops.softmax(x, layout, 16, flag_fused=flag_fused)
    assert isinstance(out, bs.BlksprsTensor) and out.shape == (0, 16, 16)


def test_oversized_rows_fall_back_and_fused_entry_point_raises(device):
    # reference: test_regressions.py:1758-1791 - 8193 blocks of 16 pad to 16384 * 16 > 131072 elements
    sbs, n = 16, 8193
    layout = torch.ones((1, 1, n), dtype=torch.bool, device=device)
    x = torch.zeros((n, sbs, sbs), device=device)
    cache = {}
    out = bs.ops.softmax(x, layout, sbs, layout_cache=cache)
    assert torch.allclose(out, torch.full_like(out, 1.0 / (n * sbs)), rtol=1e-5, atol=0)
    for key in ("packed_indices_sorted", "max_blocks_line", "layout_indices", "packed_indices_rws"):
        assert key in cache
    assert cache["max_blocks_line"] == 16384
    with pytest.raises(ValueError, match="131072"):
        bs.ops.softmax_fused(x, layout, sbs)
    regular = bs.ops.softmax(x, layout, sbs, flag_fused=False)
    assert torch.equal(regular, out)


def test_rejects_other_dtypes(device):
    layout = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    with pytest.raises(ValueError, match="Tensor must have float32 dtype"):
        bs.ops.softmax(torch.randn((1, 16, 16), device=device, dtype=torch.float16), layout, 16)
