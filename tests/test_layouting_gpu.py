"""Bit-exact parity of the data-dependent layout builders with the CPU oracle.

``build_sparsity_layout`` follows the reference's own tests: a to_dense round trip gives the layout back
(test/cases/test_blocksparse.py:990-1009), NaN activates a block (test/cases/test_regressions.py:1943-1980),
sizes that the block size does not divide are rejected (test/cases/test_blocksparse.py:1073-1080)."""

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import rand_layout

pytestmark = pytest.mark.gpu

DTYPES = [torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64,
          torch.float16, torch.bfloat16, torch.float32, torch.float64]


def _sparse_dense(shape, sbs, dtype, seed, density=0.4):
    """Dense tensor with whole blocks zeroed, one surviving element in some of the kept blocks only."""
    g = torch.Generator().manual_seed(seed)
    B, R, C = shape
    keep = rand_layout(shape, density, seed=seed + 1)
    if dtype == torch.bool:
        x = torch.rand((B, R * sbs, C * sbs), generator=g) < 0.5
    elif dtype.is_floating_point:
        x = torch.randn((B, R * sbs, C * sbs), generator=g).to(dtype)
    else:
        x = torch.randint(-100 if dtype != torch.uint8 else 0, 100, (B, R * sbs, C * sbs), generator=g).to(dtype)
    mask = keep.repeat_interleave(sbs, 1).repeat_interleave(sbs, 2)
    x = torch.where(mask, x, torch.zeros((), dtype=dtype))
    # a block whose only non-zero element sits in its last row and column
    lone = (~keep).nonzero()
    if lone.numel():
        b, r, c = lone[0].tolist()
        x[b, r * sbs + sbs - 1, c * sbs + sbs - 1] = True if dtype == torch.bool else 1
    return x


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sbs,shape", [(16, (2, 3, 5)), (32, (3, 4, 2)), (64, (1, 2, 9)), (128, (1, 2, 1)), (16, (1, 1, 300))])
def test_layout_of_a_dense_tensor_all_dtypes(device, dtype, sbs, shape):
    x = _sparse_dense(shape, sbs, dtype, seed=sbs + shape[2])
    got = bs.layouting.build_sparsity_layout(x.to(device), sbs)
    assert type(got) is torch.Tensor and got.dtype == torch.bool and got.shape == shape
    assert torch.equal(got.cpu(), torch.from_numpy(orc.build_sparsity_layout(x, sbs)))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32, torch.float64])
def test_nan_activates_a_block_and_negative_zero_does_not(device, dtype):
    sbs = 16
    dense = torch.zeros((1, sbs, 3 * sbs), dtype=dtype, device=device)
    dense[0, 0, sbs] = float("nan")
    dense[0, 5, 2 * sbs + 7] = -0.0
    assert torch.equal(bs.layouting.build_sparsity_layout(dense, sbs).cpu(), torch.tensor([[[False, True, False]]]))
    dense[0, 15, 2 * sbs + 15] = float("-inf")
    assert torch.equal(bs.layouting.build_sparsity_layout(dense, sbs).cpu(), torch.tensor([[[False, True, True]]]))


def test_round_trip_through_to_dense_gives_the_layout_back(device):
    for sbs, shape, seed in ((16, (2, 4, 4), 0), (64, (2, 3, 5), 1)):
        layout = rand_layout(shape, 0.5, seed=seed).to(device)
        g = torch.Generator(device=device).manual_seed(seed)
        x = torch.randn((shape[0], shape[1] * sbs, shape[2] * sbs), generator=g, device=device)
        blocks = bs.ops.to_sparse(x, layout, sbs)
        dense = bs.ops.to_dense(blocks, layout, sbs)
        assert torch.equal(bs.layouting.build_sparsity_layout(dense, sbs), layout.bool())
        with torch.amp.autocast(device_type="cuda", enabled=True):
            assert torch.equal(bs.layouting.build_sparsity_layout(dense, sbs), layout.bool())
    full = bs.layouting.build_sparsity_layout_full(x, 64)
    assert full.dtype == torch.bool and full.shape == (2, 3, 5) and bool(full.all())


def test_non_contiguous_input_empty_input_and_errors(device):
    x = torch.randn((2, 64, 32), device=device).transpose(1, 2)  # (2, 32, 64), not contiguous
    assert torch.equal(bs.layouting.build_sparsity_layout(x, 16).cpu(),
                       torch.from_numpy(orc.build_sparsity_layout(x.cpu().contiguous(), 16)))
    assert bs.layouting.build_sparsity_layout(torch.zeros((0, 32, 32), device=device), 16).shape == (0, 2, 2)
    with pytest.raises(ValueError, match="divisible"):
        bs.layouting.build_sparsity_layout(torch.zeros((1, 17, 16), device=device), 16)
    with pytest.raises(ValueError, match="divisible"):
        bs.layouting.build_sparsity_layout_full(torch.zeros((1, 17, 16), device=device), 16)
    with pytest.raises(ValueError, match="3 dimensions"):
        bs.layouting.build_sparsity_layout(torch.zeros((32, 32), device=device), 16)
    with pytest.raises(ValueError, match="GPU"):
        bs.layouting.build_sparsity_layout(torch.zeros((1, 32, 32)), 16)
    with pytest.raises(ValueError, match="at least 16"):
        bs.layouting.build_sparsity_layout(torch.zeros((1, 32, 32), device=device), 8)


def test_full_size_layout_property(device):
    """A tensor of the size of configuration 2's dense operand (16 x 4096 x 4096 bf16): the layout of
    to_dense(to_sparse(x, l), l) is l for a random l (needs no oracle at this size)."""
    sbs = 64
    layout = rand_layout((16, 64, 64), 0.25, seed=3).to(device)
    x = torch.randn((16, 4096, 4096), device=device, dtype=torch.bfloat16)
    dense = bs.ops.to_dense(bs.ops.to_sparse(x, layout, sbs), layout, sbs)
    assert torch.equal(bs.layouting.build_sparsity_layout(dense, sbs), layout.bool())
