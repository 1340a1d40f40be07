"""Bit-exact parity of the device LUT builders with the CPU oracle."""

import numpy as np
import pytest
import torch

import blksprs_amd as bs
from blksprs_amd.ops.flash_attention import _build_segmented_indices, _select_segmented_index_dtype
from blksprs_amd.ops.matmul import matmul_build_layout_cache
from blksprs_amd.ops.softmax import softmax_build_layout_cache, softmax_fused_build_layout_cache
from blksprs_amd.utils import tools
from oracle import blksprs_oracle as orc
from tests.helpers import rand_layout

pytestmark = pytest.mark.gpu

SHAPES = [((1, 1, 1), 1.0), ((1, 1, 1), 0.0), ((2, 3, 4), 0.5), ((2, 8, 8), 0.5), ((3, 5, 7), 0.2),
          ((4, 17, 33), 0.7), ((16, 64, 64), 0.25), ((2, 128, 128), 0.05), ((1, 1, 5000), 0.5),
          ((7, 300, 11), 0.9), ((2, 0, 4), 0.5), ((0, 3, 3), 0.5), ((2, 3, 0), 0.5)]


@pytest.mark.parametrize("shape,density", SHAPES)
@pytest.mark.parametrize("dtype", [torch.bool, torch.int32, torch.float16])
def test_packed_and_layout_indices(device, shape, density, dtype):
    layout = rand_layout(shape, density, seed=sum(shape))
    dev_layout = layout.to(dtype).to(device)
    packed = tools.build_packed_indices(dev_layout)
    assert packed.dtype == torch.int64 and type(packed) is torch.Tensor
    assert np.array_equal(packed.cpu().numpy(), orc.packed_indices(layout.numpy()))
    lidx = tools.build_layout_indices(dev_layout)
    assert lidx.dtype == torch.int64 and lidx.is_contiguous()
    assert np.array_equal(lidx.cpu().numpy(), orc.layout_indices(layout.numpy()))
    assert torch.equal(lidx.cpu(), torch.nonzero(layout))
    info = tools.pack_layout(dev_layout)
    assert info.count == orc.n_sparse_blocks(layout.numpy())


def test_block_count_of_large_half_precision_layout_is_exact(device):
    # 65536 ones cannot be summed in fp16 (reference: test_regressions.py:1060-1075)
    layout = torch.ones((1, 256, 256), dtype=torch.float16, device=device)
    assert tools.pack_layout(layout).count == 65536


@pytest.mark.parametrize("shape,density", SHAPES)
def test_segmented_indices(device, shape, density):
    layout = rand_layout(shape, density, seed=3 + sum(shape))
    B, R, C = shape
    indices, offsets, longest = _build_segmented_indices(layout.to(device), B, R, C)
    exp_idx, exp_off, exp_long = orc.segmented_indices(layout.numpy())
    assert indices.dtype == torch.int32 and offsets.dtype == torch.int32
    assert np.array_equal(indices.cpu().numpy(), exp_idx)
    assert np.array_equal(offsets.cpu().numpy(), exp_off)
    assert longest == exp_long
    # the transposed adjacency used by the backward pass
    lt = layout.transpose(1, 2).contiguous()
    indices, offsets, longest = _build_segmented_indices(lt.to(device), B, C, R)
    exp_idx, exp_off, exp_long = orc.segmented_indices(lt.numpy())
    assert np.array_equal(indices.cpu().numpy(), exp_idx) and np.array_equal(offsets.cpu().numpy(), exp_off)
    assert longest == exp_long


def test_segmented_index_dtype_selection():
    assert _select_segmented_index_dtype(0, 1) == torch.int32
    assert _select_segmented_index_dtype(2_147_483_647, 2_147_483_648) == torch.int32
    assert _select_segmented_index_dtype(2_147_483_648, 1) == torch.int64
    assert _select_segmented_index_dtype(1, 2_147_483_649) == torch.int64


@pytest.mark.parametrize("shape,density", [s for s in SHAPES if 0 not in s[0]])
def test_softmax_metadata(device, shape, density):
    layout = rand_layout(shape, density, seed=5 + sum(shape)).to(device)
    cache = softmax_fused_build_layout_cache(None, layout)
    exp_sorted, exp_mbl = orc.sorted_packed_indices(layout.cpu().numpy())
    assert np.array_equal(cache["packed_indices_sorted"].cpu().numpy(), exp_sorted)
    assert cache["max_blocks_line"] == exp_mbl
    # also equals the torch formulation of the reference
    ref = (torch.from_numpy(orc.packed_indices(layout.cpu().numpy())).reshape(layout.shape)
           .sort(descending=True, dim=-1)[0].reshape(-1))
    assert torch.equal(cache["packed_indices_sorted"].cpu(), ref)
    cache = softmax_build_layout_cache(cache, layout)
    assert "packed_indices_sorted" in cache  # both metadata sets share one cache
    assert torch.equal(cache["layout_indices"].cpu(), torch.nonzero(layout.cpu()))
    rws = layout.cpu().any(dim=-1, keepdim=True)
    assert np.array_equal(cache["packed_indices_rws"].cpu().numpy(), orc.packed_indices(rws.numpy()))


@pytest.mark.parametrize("dims,px,py", [((2, 8, 8, 8), 0.5, 0.5), ((1, 1, 1, 1), 1.0, 1.0), ((3, 5, 70, 9), 0.3, 0.3),
                                        ((2, 16, 130, 16), 0.1, 0.4), ((16, 64, 64, 64), 0.25, 0.25),
                                        ((2, 4, 0, 4), 0.5, 0.5), ((2, 128, 128, 128), 0.05, 0.05)])
def test_product_layout_and_contraction_lists(device, dims, px, py):
    B, R, K, C = dims
    lx = rand_layout((B, R, K), px, seed=R + K)
    ly = rand_layout((B, K, C), py, seed=K + C + 1)
    lo = bs.layouting.build_sparsity_layout_matmul(lx.to(device), ly.to(device))
    assert lo.dtype == torch.bool and type(lo) is torch.Tensor
    assert np.array_equal(lo.cpu().numpy(), orc.layout_matmul(lx.numpy(), ly.numpy()))
    # an output layout that is not the product: extra blocks get empty lists, missing ones are skipped
    lo2 = rand_layout((B, R, C), 0.6, seed=99)
    for out_layout in (lo.cpu(), lo2):
        cache = matmul_build_layout_cache(None, lx.to(device), ly.to(device), out_layout.to(device))
        exp_off, exp_pairs = orc.contraction_lists(lx.numpy(), ly.numpy(), out_layout.numpy())
        assert cache["contraction_offsets"].dtype == torch.int32
        assert np.array_equal(cache["contraction_offsets"].cpu().numpy(), exp_off)
        assert np.array_equal(cache["contraction_pairs"].cpu().numpy(), exp_pairs)
        assert np.array_equal(cache["packed_indices_x"].cpu().numpy(), orc.packed_indices(lx.numpy()))
        assert np.array_equal(cache["packed_indices_y"].cpu().numpy(), orc.packed_indices(ly.numpy()))
        assert torch.equal(cache["layout_indices_o"].cpu(), torch.nonzero(out_layout))
        assert cache["n_sparse_blocks"] == int(out_layout.sum())


def test_cached_metadata_are_plain_tensors_and_cache_invalidates(device):
    # reference: test_regressions.py:318-360, :1734-1755
    layout = rand_layout((2, 4, 4), 0.5, seed=1).to(device)
    x = torch.randn((2, 64, 64), device=device)
    cache = {}
    bs.ops.to_sparse(x, layout, 16, layout_cache=cache)
    first = cache["layout_indices"]
    assert all(type(v) is torch.Tensor for v in cache.values() if isinstance(v, torch.Tensor))
    bs.ops.to_sparse(x, layout, 16, layout_cache=cache)
    assert cache["layout_indices"] is first  # reused
    layout[0, 0, 0] = ~layout[0, 0, 0]  # in-place change bumps the version
    bs.ops.to_sparse(x, layout, 16, layout_cache=cache)
    assert cache["layout_indices"] is not first
    assert cache["n_sparse_blocks"] == int(layout.sum())
    other = rand_layout((2, 4, 4), 0.5, seed=2).to(device)
    bs.ops.to_sparse(x, other, 16, layout_cache=cache)
    assert torch.equal(cache["layout_indices"].cpu(), torch.nonzero(other.cpu()))
    # mutating a derived tensor invalidates as well
    kept = cache["layout_indices"]
    kept.add_(0)
    bs.ops.to_sparse(x, other, 16, layout_cache=cache)
    assert cache["layout_indices"] is not kept


@pytest.mark.parametrize("n_rows,rows_per_batch,parts_log2", [(1024, 64, 0), (1024, 64, 1), (21, 7, 2), (5, 5, 1),
                                                              (8, 1, 3), (3, 3, 0), (4099, 128, 0)])
def test_row_work_table_of_the_device_equals_its_restatement(device, n_rows, rows_per_batch, parts_log2):
    """``bsa_lut_row_work_table`` (keys on the device, a stable radix sort, placement by binary search) against the
    restatement in torch, bit for bit: plain, with a sweep, with long and short rows paired, and with a bound on the
    work that is far above the largest row."""
    import importlib
    from tests import helpers
    mm = importlib.import_module("blksprs_amd.ops.matmul")
    g = torch.Generator().manual_seed(n_rows + parts_log2)
    blocks_per_row = 9
    row_offsets = torch.arange(n_rows + 1, dtype=torch.int32) * blocks_per_row
    pair_offsets = torch.cumsum(torch.randint(0, 6, (n_rows * blocks_per_row + 1,), generator=g), 0).to(torch.int32)
    bound = 5 * blocks_per_row
    for pair_up, sweep, max_work in ((False, 0, bound), (False, 3, bound), (True, 0, bound), (False, 32, 1000 * bound)):
        want = helpers.expected_row_work_table(pair_offsets, row_offsets, rows_per_batch, parts_log2, pair_up,
                                               max_work=max_work, sweep=sweep)
        got = mm._row_work_table(pair_offsets.to(device), row_offsets.to(device), rows_per_batch, parts_log2, pair_up,
                                 max_work=max_work, sweep=sweep)
        assert got.dtype == torch.int32 and torch.equal(got.cpu(), want), (pair_up, sweep)
    # many rows of equal work keep their order (the sort is stable)
    flat = torch.arange(n_rows * blocks_per_row + 1, dtype=torch.int32) * 2
    want = helpers.expected_row_work_table(flat, row_offsets, rows_per_batch, parts_log2, max_work=2 * blocks_per_row)
    got = mm._row_work_table(flat.to(device), row_offsets.to(device), rows_per_batch, parts_log2,
                             max_work=2 * blocks_per_row)
    assert torch.equal(got.cpu(), want)
    # no rows: an empty table, nothing launched
    assert mm._row_work_table(torch.zeros(1, dtype=torch.int32, device=device),
                              torch.zeros(1, dtype=torch.int32, device=device), 1, 1).numel() == 0


@pytest.mark.parametrize("shape,density", [((3, 40, 37), 0.3), ((1, 5, 130), 0.9), ((2, 64, 64), 0.02), ((1, 1, 1), 1.0)])
def test_block_order_of_the_device_equals_its_restatement(device, shape, density):
    """``bsa_lut_block_order`` against the stable argsort of the same key in torch, and as a permutation."""
    import importlib
    from tests import helpers
    mm = importlib.import_module("blksprs_amd.ops.matmul")
    layout = rand_layout(shape, density, 11, ensure_rows=True)
    coords = torch.nonzero(layout)
    got = mm._block_order(coords.to(device), shape[1], shape[2]).cpu()
    want = helpers.expected_block_order(coords, shape[1], shape[2])
    assert got.dtype == torch.int32 and torch.equal(got, want)
    assert torch.equal(torch.sort(got.long())[0], torch.arange(coords.size(0)))
    assert mm._block_order(torch.empty((0, 3), dtype=torch.int64, device=device), 4, 4).numel() == 0


@pytest.mark.parametrize("shape,density", [((3, 40, 37), 0.3), ((2, 5, 130), 0.9), ((2, 64, 64), 0.02), ((1, 1, 1), 1.0),
                                           ((2, 7, 9), 0.0), ((4, 9, 300), 0.5)])
def test_pair_lists_of_the_device_equal_their_restatement(device, shape, density):
    """``bsa_lut_pair_union`` / ``bsa_lut_pair_entries`` through the C ABI against the same lists formed in numpy:
    the union of rows 2 g and 2 g + 1 (a lone last row with nothing), and per active position of the union, in
    row-major order, column | first row active << 28 | second row active << 29."""
    from blksprs_amd import _capi
    B, R, C = shape
    G = (R + 1) // 2
    layout = rand_layout(shape, density, seed=3 + sum(shape)).to(torch.uint8)
    padded = np.zeros((B, 2 * G, C), dtype=np.uint8)
    padded[:, :R] = layout.numpy()
    first, second = padded[:, 0::2], padded[:, 1::2]
    want_union = first | second
    where = np.nonzero(want_union.reshape(-1))[0]
    want_entries = ((where % C) | (first.reshape(-1)[where].astype(np.int64) << 28)
                    | (second.reshape(-1)[where].astype(np.int64) << 29)).astype(np.int32)

    dev_layout = layout.to(device)
    uni = torch.full((B, G, C), 7, dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    _capi.call("bsa_lut_pair_union", dev_layout.data_ptr(), B, R, C, uni.data_ptr(), stream)
    assert np.array_equal(uni.cpu().numpy(), want_union)
    packed = tools.build_packed_indices(uni)
    entries = torch.full((max(len(where), 1),), -5, dtype=torch.int32, device=device)
    _capi.call("bsa_lut_pair_entries", dev_layout.data_ptr(), packed.data_ptr(), B, R, C, entries.data_ptr(), stream)
    assert np.array_equal(entries.cpu().numpy()[:len(where)], want_entries)
    if len(where) == 0:
        assert int(entries[0]) == -5  # nothing written
