"""Bit-exact parity of to_sparse / to_dense with the CPU oracle, all supported dtypes."""

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import rand_layout

pytestmark = pytest.mark.gpu

DTYPES = [torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64,
          torch.float16, torch.bfloat16, torch.float32, torch.float64]


def _dense(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype == torch.bool:
        return torch.rand(shape, generator=g) < 0.5
    if dtype.is_floating_point:
        return torch.randn(shape, generator=g).to(dtype)
    info = torch.iinfo(dtype)
    return torch.randint(max(info.min, -1000), min(info.max, 1000), shape, generator=g).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sbs,shape", [(16, (2, 3, 5)), (32, (3, 4, 2)), (64, (1, 2, 3)), (128, (1, 2, 1))])
def test_round_trip_all_dtypes(device, dtype, sbs, shape):
    layout = rand_layout(shape, 0.5, seed=sbs, ensure_rows=True)
    B, R, C = shape
    x = _dense((B, R * sbs, C * sbs), dtype, seed=sbs + 1)
    blocks = bs.ops.to_sparse(x.to(device), layout.to(device), sbs)
    assert isinstance(blocks, bs.BlksprsTensor) and blocks.dtype == dtype
    assert torch.equal(blocks.cpu(), orc.to_sparse(x, layout.numpy(), sbs))
    fill = True if dtype == torch.bool else 3
    dense = bs.ops.to_dense(blocks, layout.to(device), sbs, fill_value=fill)
    assert type(dense) is torch.Tensor and dense.dtype == dtype
    assert torch.equal(dense.cpu(), orc.to_dense(orc.to_sparse(x, layout.numpy(), sbs), layout.numpy(), sbs, fill))


def test_fill_values_and_aliases(device):
    sbs = 16
    layout = rand_layout((2, 4, 4), 0.4, seed=1)
    x = torch.randn((2, 64, 64))
    blocks = bs.ops.to_blksprs(x.to(device), layout.to(device), sbs)
    for fill in (0, -1.5, float("-inf"), float("nan")):
        got = bs.ops.from_blksprs(blocks, layout.to(device), sbs, fill_value=fill).cpu()
        exp = orc.to_dense(orc.to_sparse(x, layout.numpy(), sbs), layout.numpy(), sbs, fill)
        assert torch.equal(torch.nan_to_num(got, nan=123.0), torch.nan_to_num(exp, nan=123.0))
    assert torch.equal(bs.ops.to_sparse_shaped(x.to(device), layout.to(device), sbs).cpu(), blocks.cpu())
    assert torch.equal(bs.ops.to_dense_shaped(blocks, layout.to(device), sbs).cpu(),
                       bs.ops.to_dense(blocks, layout.to(device), sbs).cpu())


def test_single_block_layout_aliases_input(device):
    # reference: test_regressions.py:1312-1324
    layout = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    x = torch.randn((1, 16, 16), device=device, requires_grad=True)
    blocks = bs.ops.to_sparse(x, layout, 16)
    dense = bs.ops.to_dense(blocks, layout, 16)
    assert type(dense) is torch.Tensor
    assert dense.data_ptr() == x.data_ptr()
    dense.sum().backward()
    assert torch.equal(x.grad, torch.ones_like(x))


def test_empty_and_ragged_layouts(device):
    sbs = 16
    # no active block at all
    layout = torch.zeros((2, 2, 3), dtype=torch.bool, device=device)
    x = torch.randn((2, 32, 48), device=device)
    blocks = bs.ops.to_sparse(x, layout, sbs)
    assert blocks.shape == (0, sbs, sbs)
    assert torch.all(bs.ops.to_dense(blocks, layout, sbs, fill_value=2.0) == 2.0)
    # a batch without blocks next to a full one
    layout = torch.zeros((2, 2, 2), dtype=torch.bool)
    layout[1] = True
    x = torch.randn((2, 32, 32))
    blocks = bs.ops.to_sparse(x.to(device), layout.to(device), sbs)
    assert torch.equal(blocks.cpu(), orc.to_sparse(x, layout.numpy(), sbs))


def test_conversions_are_each_others_gradient(device):
    sbs = 32
    layout = rand_layout((2, 3, 3), 0.5, seed=4)
    x = torch.randn((2, 96, 96), device=device, requires_grad=True)
    blocks = bs.ops.to_sparse(x, layout.to(device), sbs)
    w = torch.randn_like(blocks)
    (blocks * w).sum().backward()
    assert torch.equal(x.grad.cpu(), orc.to_dense(w.cpu(), layout.numpy(), sbs))
    b = torch.randn((int(layout.sum()), sbs, sbs), device=device, requires_grad=True)
    dense = bs.ops.to_dense(b, layout.to(device), sbs)
    wd = torch.randn_like(dense)
    (dense * wd).sum().backward()
    assert torch.equal(b.grad.cpu(), orc.to_sparse(wd.cpu(), layout.numpy(), sbs))


def test_full_size_round_trip_property(device):
    """Config 5's conversion leg at full size: to_dense(to_sparse(X)) equals X on active blocks and the fill
    value elsewhere (checked on the device, no oracle needed)."""
    sbs, B, n = 16, 64, 128
    layout = rand_layout((B, n, n), 0.05, seed=0, ensure_rows=True).to(device)
    x = torch.randn((B, n * sbs, n * sbs), device=device, dtype=torch.float16)
    blocks = bs.ops.to_sparse(x, layout, sbs)
    assert blocks.size(0) == int(layout.sum())
    dense = bs.ops.to_dense(blocks, layout, sbs, fill_value=-2.0)
    active = layout.repeat_interleave(sbs, 1).repeat_interleave(sbs, 2)
    assert torch.equal(dense[active], x[active])
    assert torch.all(dense[~active] == -2.0)
    assert torch.equal(bs.ops.to_sparse(dense, layout, sbs), blocks)


def test_validation_errors(device):
    layout = torch.ones((1, 2, 2), dtype=torch.bool, device=device)
    with pytest.raises(ValueError, match="Tensor must have 3 dimensions"):
        bs.ops.to_sparse(torch.randn((32, 32), device=device), layout, 16)
    with pytest.raises(ValueError, match="Tensors must be on GPU"):
        bs.ops.to_sparse(torch.randn((1, 32, 32)), layout, 16)
    with pytest.raises(ValueError, match="batch dimension"):
        bs.ops.to_sparse(torch.randn((2, 32, 32), device=device), layout, 16)
    with pytest.raises(ValueError, match="at least 16"):
        bs.ops.to_sparse(torch.randn((1, 16, 16), device=device), layout, 8)
    with pytest.raises(ValueError, match="power of 2"):
        bs.ops.to_sparse(torch.randn((1, 48, 48), device=device), layout, 24)
    with pytest.raises(ValueError, match="Mismatch between sparsity layout and blocks"):
        bs.ops.to_dense(torch.randn((3, 16, 16), device=device), layout, 16)
    with pytest.raises(ValueError, match="0 or 1"):
        bs.ops.to_dense(torch.randn((4, 16, 16), device=device), layout.float() * 2, 16)
    with pytest.raises(ValueError, match="complex dtype"):
        bs.ops.to_dense(torch.randn((4, 16, 16), device=device), layout.to(torch.complex64), 16)
    with pytest.raises(ValueError, match="not supported"):
        bs.ops.to_sparse(torch.randn((1, 32, 32), device=device).to(torch.complex64), layout, 16)
