"""Bit-exact parity of ``bs.ops.transpose`` with the CPU oracle, its gradient, cache keys and error behaviour.

Modelled on the reference's tests: dense transpose through a conversion round trip with gradients
(test/cases/test_blocksparse.py:204-239), every supported dtype keeps its dtype
(test/cases/test_regressions.py:1399-1434), returned layouts are plain tensors (:1688-1712)."""

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import rand_layout

pytestmark = pytest.mark.gpu

DTYPES = [torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64,
          torch.float16, torch.bfloat16, torch.float32, torch.float64]


def _blocks(n, sbs, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype == torch.bool:
        return torch.rand((n, sbs, sbs), generator=g) < 0.5
    if dtype.is_floating_point:
        return torch.randn((n, sbs, sbs), generator=g).to(dtype)
    return torch.randint(0 if dtype == torch.uint8 else -100, 100, (n, sbs, sbs), generator=g).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sbs,shape", [(16, (2, 3, 5)), (32, (3, 4, 2)), (64, (2, 5, 3)), (128, (1, 2, 3)), (256, (1, 1, 2))])
def test_transpose_all_dtypes(device, dtype, sbs, shape):
    layout = rand_layout(shape, 0.6, seed=sbs + 7)
    x = _blocks(int(layout.sum()), sbs, dtype, seed=sbs)
    got, layout_t = bs.ops.transpose(x.to(device), layout.to(device), sbs)
    exp, exp_layout = orc.transpose(x, layout.numpy(), sbs)
    assert isinstance(got, bs.BlksprsTensor) and got.dtype == dtype
    assert type(layout_t) is torch.Tensor and layout_t.is_contiguous()
    assert torch.equal(layout_t.cpu().bool(), torch.from_numpy(exp_layout))
    assert torch.equal(got.cpu().as_subclass(torch.Tensor), exp)


def test_dense_transpose_through_a_round_trip_with_gradients(device):
    for sbs, (b, m, k), density in ((16, (2, 64, 32), 0.5), (64, (2, 128, 256), 0.4), (32, (1, 32, 96), 1.0)):
        for use_amp in (False, True):
            with torch.amp.autocast(device_type="cuda", enabled=use_amp):
                layout = rand_layout((b, m // sbs, k // sbs), density, seed=m).to(device)
                g = torch.Generator(device=device).manual_seed(k)
                x_d = torch.randn((b, m, k), generator=g, device=device)
                x_d = bs.ops.to_dense(bs.ops.to_sparse(x_d, layout, sbs), layout, sbs)
                x_stock = x_d.clone().requires_grad_(True)
                x_ours = x_d.clone().requires_grad_(True)
                stock = x_stock.transpose(1, 2)
                out, layout_t = bs.ops.transpose(bs.ops.to_sparse(x_ours, layout, sbs), layout, sbs)
                dense = bs.ops.to_dense(out, layout_t, sbs)
                assert torch.equal(dense, stock)
                target = torch.randn_like(stock)
                torch.nn.L1Loss()(stock, target).backward()
                torch.nn.L1Loss()(dense, target).backward()
                # the gradient only exists on active blocks: compare there
                mask = layout.bool().repeat_interleave(sbs, 1).repeat_interleave(sbs, 2)
                assert torch.equal(x_ours.grad, torch.where(mask, x_stock.grad, torch.zeros_like(x_stock.grad)))


def test_cache_keys_reuse_and_empty_layouts(device):
    sbs = 16
    layout = rand_layout((2, 3, 4), 0.5, seed=1).to(device)
    x = torch.randn((int(layout.sum()), sbs, sbs), device=device)
    cache = {}
    out1, lt1 = bs.ops.transpose(x, layout, sbs, layout_cache=cache)
    for key in ("sparsity_layout_t", "layout_indices", "packed_indices", "n_sparse_blocks"):
        assert key in cache
    assert cache["n_sparse_blocks"] == int(layout.sum())
    assert torch.equal(cache["layout_indices"].cpu(), torch.nonzero(layout.transpose(1, 2).contiguous()).cpu())
    ids = {k: id(cache[k]) for k in ("sparsity_layout_t", "layout_indices", "packed_indices")}
    out2, lt2 = bs.ops.transpose(x, layout, sbs, layout_cache=cache)
    assert torch.equal(out1, out2) and lt2 is lt1
    assert all(id(cache[k]) == v for k, v in ids.items())
    # twice is the identity
    back, layout_back = bs.ops.transpose(out1, lt1, sbs)
    assert torch.equal(back, x) and torch.equal(layout_back.bool(), layout.bool())
    # nothing active
    empty = torch.zeros((1, 2, 3), dtype=torch.bool, device=device)
    out, lt = bs.ops.transpose(torch.empty((0, sbs, sbs), device=device), empty, sbs)
    assert out.shape == (0, sbs, sbs) and lt.shape == (1, 3, 2)
    # a square layout that equals its transpose still gets storage of its own
    sym = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    _, lt = bs.ops.transpose(torch.randn((1, sbs, sbs), device=device), sym, sbs)
    assert lt.data_ptr() != sym.data_ptr()


def test_validation_errors(device):
    sbs = 16
    layout = torch.ones((1, 1, 2), dtype=torch.bool, device=device)
    with pytest.raises(ValueError, match="dtype is not supported"):
        bs.ops.transpose(torch.zeros((2, sbs, sbs), dtype=torch.complex64, device=device), layout, sbs)
    with pytest.raises(ValueError, match="3 dimensions"):
        bs.ops.transpose(torch.zeros((sbs, sbs), device=device), layout, sbs)
    with pytest.raises(ValueError, match="GPU"):
        bs.ops.transpose(torch.zeros((2, sbs, sbs)), layout, sbs)
    with pytest.raises(ValueError):
        bs.ops.transpose(torch.zeros((3, sbs, sbs), device=device), layout, sbs)  # block count mismatch


def test_full_size_property(device):
    """Configuration 2's x operand (bf16, B=16, 64 x 64 blocks of 64, 25 %): transposing twice is the identity
    and one transposition agrees with the dense transpose on a sampled batch entry."""
    sbs = 64
    layout = rand_layout((16, 64, 64), 0.25, seed=0).to(device)
    x = torch.randn((int(layout.sum()), sbs, sbs), device=device, dtype=torch.bfloat16)
    out, layout_t = bs.ops.transpose(x, layout, sbs)
    back, _ = bs.ops.transpose(out, layout_t, sbs)
    assert torch.equal(back, x)
    dense = bs.ops.to_dense(x, layout, sbs)
    dense_t = bs.ops.to_dense(out, layout_t, sbs)
    assert torch.equal(dense_t[5], dense[5].transpose(0, 1))
