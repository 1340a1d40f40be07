"""Parity of the block-sparse matmul with the CPU oracle: rtol = atol = 1e-5 for fp32, 2e-2 for fp16 / bf16
against an fp32-accumulated dense-masked product of the rounded inputs."""

import math

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import assert_close, rand_blocks, rand_layout

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def _problem(B, R, K, C, sbs, dtype, density, seed, product_layout=True):
    lx = rand_layout((B, R, K), density, seed=seed, ensure_rows=True)
    ly = rand_layout((B, K, C), density, seed=seed + 1, ensure_rows=True)
    if product_layout:
        lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
    else:
        lo = rand_layout((B, R, C), 0.6, seed=seed + 2)
    scale = 1.0 / math.sqrt(K * sbs)
    x = rand_blocks(int(lx.sum()), sbs, dtype, seed + 3, scale)
    y = rand_blocks(int(ly.sum()), sbs, dtype, seed + 4)
    return lx, ly, lo, x, y


def _oracle(x, lx, y, ly, lo, sbs):
    # fp64 accumulation of the (already rounded) inputs is the tightest statement of "fp32-accumulated"
    return orc.matmul(x.double(), lx.numpy(), y.double(), ly.numpy(), lo.numpy(), sbs, acc_dtype=torch.float64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sbs,dims,density", [
    (32, (2, 8, 8, 8), 0.5),      # config 1: B=2, 256^3, sbs 32, p = 0.5
    (16, (3, 5, 9, 6), 0.4),
    (16, (2, 16, 16, 16), 0.1),
    (32, (2, 3, 7, 5), 0.6),
    (64, (2, 4, 6, 5), 0.5),
    (64, (1, 3, 20, 3), 0.9),
    (128, (1, 2, 3, 2), 0.7),
    (256, (1, 1, 2, 1), 1.0),
])
def test_forward_matches_oracle(device, dtype, sbs, dims, density):
    B, R, K, C = dims
    for product_layout in (True, False):
        lx, ly, lo, x, y = _problem(B, R, K, C, sbs, dtype, density, seed=sbs + K, product_layout=product_layout)
        out = bs.ops.matmul(x.to(device), lx.to(device), y.to(device), ly.to(device), lo.to(device), sbs)
        assert isinstance(out, bs.BlksprsTensor) and out.dtype == dtype
        assert out.shape == (int(lo.sum()), sbs, sbs)
        assert_close(out, _oracle(x, lx, y, ly, lo, sbs), TOL[dtype], f"matmul {dtype} sbs={sbs} product={product_layout}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sbs", [16, 32, 64, 128])
def test_backward_matches_autograd_of_the_oracle(device, dtype, sbs):
    B, R, K, C = 2, 3, 4, 5
    lx, ly, lo, x, y = _problem(B, R, K, C, sbs, dtype, 0.6, seed=sbs)
    xg = x.to(device).requires_grad_(True)
    yg = y.to(device).requires_grad_(True)
    cache = {}
    lxd, lyd, lod = lx.to(device), ly.to(device), lo.to(device)
    out = bs.ops.matmul(xg, lxd, yg, lyd, lod, sbs, layout_cache=cache)
    # the upstream gradient is scaled like the forward operands of config 2 (1 / sqrt of the contraction
    # length), so the gradients are O(1) like the operands and the stated tolerances apply to them as they are
    go = rand_blocks(out.size(0), sbs, dtype, seed=9, scale=1.0 / math.sqrt(C * sbs))
    out.backward(go.to(device))
    x64 = x.double().requires_grad_(True)
    y64 = y.double().requires_grad_(True)
    xd = orc.to_dense_autograd(x64, lx.numpy(), sbs)
    yd = orc.to_dense_autograd(y64, ly.numpy(), sbs)
    ref = orc.to_sparse_autograd(xd @ yd, lo.numpy(), sbs)
    ref.backward(go.double())
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert_close(xg.grad, x64.grad, tol, f"dX {dtype} sbs={sbs}")
    assert_close(yg.grad, y64.grad, tol, f"dY {dtype} sbs={sbs}")
    # a second step reuses the forward and backward lists
    # (16-bit operands with 64 x 64 blocks run by lines of dO and keep part offsets instead of pair lists)
    key = "grad_x_part_table" if "grad_x_part_table" in cache else "grad_x_pair_offsets"
    assert (key == "grad_x_part_table") == (sbs == 64 and dtype != torch.float32)
    offsets = cache[key]
    xg.grad = None
    bs.ops.matmul(xg, lxd, yg, lyd, lod, sbs, layout_cache=cache).backward(go.to(device))
    assert cache[key] is offsets
    if key == "grad_x_part_table":
        assert int(cache["grad_lines_error"][0].item()) == 0
    assert_close(xg.grad, x64.grad, tol, "dX second step")


def test_config1_fp32_unscaled_normal_values(device):
    """Config 1 as stated: fp32, B=2, M=K=N=256, sbs 32, Bernoulli(0.5) layouts with one block per row
    guaranteed, product output layout, N(0,1) values; rtol = atol = 1e-5 against the fp32-accumulated
    dense-masked product (diagnosed against fp64 as well, at 2e-5)."""
    sbs, B, n = 32, 2, 8
    lx = rand_layout((B, n, n), 0.5, seed=0, ensure_rows=True)
    ly = rand_layout((B, n, n), 0.5, seed=1, ensure_rows=True)
    lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
    x = rand_blocks(int(lx.sum()), sbs, torch.float32, 2)
    y = rand_blocks(int(ly.sum()), sbs, torch.float32, 3)
    out = bs.ops.matmul(x.to(device), lx.to(device), y.to(device), ly.to(device), lo.to(device), sbs)
    fp32 = orc.matmul(x, lx.numpy(), y, ly.numpy(), lo.numpy(), sbs, acc_dtype=torch.float32)
    assert_close(out, fp32, 1e-5, "config 1 vs fp32-accumulated oracle")
    assert_close(out, _oracle(x, lx, y, ly, lo, sbs), 2e-5, "config 1 vs fp64 oracle")


def test_output_blocks_without_contributions_are_zero(device):
    sbs = 64
    lx = torch.zeros((1, 2, 2), dtype=torch.bool)
    lx[0, 0, 0] = True
    ly = torch.zeros((1, 2, 2), dtype=torch.bool)
    ly[0, 1, 1] = True
    lo = torch.ones((1, 2, 2), dtype=torch.bool)
    x = torch.randn((1, sbs, sbs), device=device, dtype=torch.bfloat16)
    y = torch.randn((1, sbs, sbs), device=device, dtype=torch.bfloat16)
    out = bs.ops.matmul(x, lx.to(device), y, ly.to(device), lo.to(device), sbs)
    assert out.shape == (4, sbs, sbs) and torch.all(out == 0)


def test_full_size_config2_linearity_and_sampled_parity(device):
    """Config 2 (bf16, B=16, 4096^3, sbs 64, 25 % density, product layout) at full size: sampled output
    blocks against the oracle, and exactness properties that need no oracle (x -> 2x doubles the result
    bit for bit; zeroing y zeroes the output)."""
    B, n, sbs = 16, 64, 64
    lx = rand_layout((B, n, n), 0.25, seed=0)
    ly = rand_layout((B, n, n), 0.25, seed=1)
    lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
    g = torch.Generator().manual_seed(2)
    x = (torch.randn((int(lx.sum()), sbs, sbs), generator=g) / 64.0).to(torch.bfloat16)
    y = torch.randn((int(ly.sum()), sbs, sbs), generator=g).to(torch.bfloat16)
    xd, yd = x.to(device), y.to(device)
    cache = {}
    lxd, lyd, lod = lx.to(device), ly.to(device), lo.to(device)
    out = bs.ops.matmul(xd, lxd, yd, lyd, lod, sbs, layout_cache=cache)
    assert out.shape[0] == int(lo.sum())
    pairs = cache["contraction_pairs"]
    doubled = bs.ops.matmul(xd * 2, lxd, yd, lyd, lod, sbs, layout_cache=cache)
    assert cache["contraction_pairs"] is pairs
    assert torch.equal(doubled, out * 2)
    zero = bs.ops.matmul(xd, lxd, torch.zeros_like(yd), lyd, lod, sbs, layout_cache=cache)
    assert torch.all(zero == 0)
    # batch 3 against the oracle (one batch keeps the dense CPU product small)
    b = 3
    sl = lambda lay, t: t[int(lay[:b].sum()):int(lay[:b + 1].sum())]
    exp = _oracle(sl(lx, x), lx[b:b + 1], sl(ly, y), ly[b:b + 1], lo[b:b + 1], sbs)
    assert_close(sl(lo, out), exp, 2e-2, "config 2, batch 3")


def test_full_size_config5_sampled_parity_and_identical_rerun(device):
    """Config 5 (fp16, B=64, 2048^3, sbs 16, 5 % density with at least one block per row, product layout) at
    full size: the sbs-16 kernel with its 32 000 waves and per-XCD partition of the runs.  One batch entry
    against the oracle, a second run bit for bit, x -> 2x exactly, and the bit-exact to_sparse / to_dense round
    trip the configuration names, on the same tensors."""
    B, n, sbs = 64, 128, 16
    lx = rand_layout((B, n, n), 0.05, seed=0, ensure_rows=True)
    ly = rand_layout((B, n, n), 0.05, seed=1, ensure_rows=True)
    lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
    g = torch.Generator().manual_seed(2)
    x = (torch.randn((int(lx.sum()), sbs, sbs), generator=g) / 8.0).to(torch.float16)
    y = torch.randn((int(ly.sum()), sbs, sbs), generator=g).to(torch.float16)
    xd, yd = x.to(device), y.to(device)
    lxd, lyd, lod = lx.to(device), ly.to(device), lo.to(device)
    cache = {}
    out = bs.ops.matmul(xd, lxd, yd, lyd, lod, sbs, layout_cache=cache)
    assert out.shape == (int(lo.sum()), sbs, sbs)
    assert torch.equal(bs.ops.matmul(xd, lxd, yd, lyd, lod, sbs, layout_cache=cache), out)
    # x -> 2x doubles every sum exactly; a result below fp16's normal range is rounded at a fixed spacing, so its
    # double may differ in the last bit: those elements are held to that spacing
    doubled = bs.ops.matmul(xd * 2, lxd, yd, lyd, lod, sbs, layout_cache=cache)
    normal = out.abs() >= 2.0 ** -13
    assert torch.equal(doubled[normal], (out * 2)[normal])
    assert (doubled.float() - 2 * out.float()).abs().max() <= 2.0 ** -24
    sl = lambda lay, t, b: t[int(lay[:b].sum()):int(lay[:b + 1].sum())]
    for b in (0, 37, 63):
        exp = _oracle(sl(lx, x, b), lx[b:b + 1], sl(ly, y, b), ly[b:b + 1], lo[b:b + 1], sbs)
        assert_close(sl(lo, out, b), exp, 2e-2, f"config 5, batch {b}")
    dense = bs.ops.to_dense(out, lod, sbs)
    assert torch.equal(bs.ops.to_sparse(dense, lod, sbs), out)
    assert torch.equal(bs.layouting.build_sparsity_layout(bs.ops.to_dense(xd, lxd, sbs), sbs), lxd.to(torch.bool))


def test_autocast_and_validation(device):
    sbs = 16
    layout = torch.ones((1, 2, 2), dtype=torch.bool, device=device)
    x = torch.randn((4, sbs, sbs), device=device)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = bs.ops.matmul(x, layout, x, layout, layout, sbs)
    assert out.dtype == torch.bfloat16
    # fp64 is not silently downcast (reference: test_regressions.py:694-722)
    with torch.autocast("cuda", dtype=torch.float16):
        with pytest.raises(ValueError, match="float16, bfloat16, or float32"):
            bs.ops.matmul(x.double(), layout, x.double(), layout, layout, sbs)
    with pytest.raises(ValueError, match="same dtype"):
        bs.ops.matmul(x, layout, x.half(), layout, layout, sbs)
    with pytest.raises(ValueError, match="Inner dimensions"):
        bs.ops.matmul(x, layout, torch.randn((6, sbs, sbs), device=device),
                      torch.ones((1, 3, 2), dtype=torch.bool, device=device), layout, sbs)
    with pytest.raises(ValueError, match="Batch dimensions"):
        bs.ops.matmul(x, layout, torch.randn((8, sbs, sbs), device=device),
                      torch.ones((2, 2, 2), dtype=torch.bool, device=device), layout, sbs)
    with pytest.raises(ValueError, match="Output sparsity layout shape"):
        bs.ops.matmul(x, layout, x, layout, torch.ones((1, 2, 3), dtype=torch.bool, device=device), sbs)
    bs.utils.disable_validation()
    try:
        out = bs.ops.matmul(x, layout, x, layout, layout, sbs)  # no checks, same result path
        assert out.shape == (4, sbs, sbs)
    finally:
        bs.utils.enable_validation()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dims,dx,dy,do", [
    ((2, 3, 40, 5), 0.9, 0.5, 0.8),     # rows with more than 16 x blocks: the part that does not fit in LDS
    ((1, 2, 6, 600), 0.5, 0.5, 0.9),    # more than 64 output blocks per wave: boundary window reloads
    ((1, 1, 30, 40), 1.0, 1.0, 1.0),    # more than 64 pairs per wave: pair window reloads
    ((3, 9, 7, 11), 0.3, 0.3, 0.5),     # empty rows, output blocks without pairs
])
def test_row_panel_kernel_is_bit_identical_to_the_tile_kernel(device, dtype, dims, dx, dy, do):
    """fp16 / bf16 with sbs 64 run the row-panel kernel; it must reproduce the per-tile kernel bit for bit
    (same pairs, same ascending-k accumulation)."""
    from blksprs_amd import _capi
    B, R, K, C = dims
    sbs = 64
    lx = rand_layout((B, R, K), dx, seed=1).to(device)
    ly = rand_layout((B, K, C), dy, seed=2).to(device)
    lo = rand_layout((B, R, C), do, seed=3).to(device)
    if dx < 0.5:
        lx[0, 0] = False  # a row without x blocks
    x = rand_blocks(int(lx.sum()), sbs, dtype, 4, 1.0 / math.sqrt(K * sbs)).to(device)
    y = rand_blocks(int(ly.sum()), sbs, dtype, 5).to(device)
    cache = {}
    out = bs.ops.matmul(x, lx, y, ly, lo, sbs, layout_cache=cache)
    ref = torch.empty_like(out)
    _capi.call("bsa_matmul", x.data_ptr(), y.data_ptr(), ref.data_ptr(), cache["contraction_offsets"].data_ptr(),
               _capi.ptr(cache["contraction_pairs"]), cache["block_order"].data_ptr(), out.size(0), x.size(0),
               y.size(0), sbs, _capi.DTYPE_CODES[dtype], 0, 0, _capi.stream(device))
    assert torch.equal(out, ref)
    assert_close(out, _oracle(x.cpu(), lx.cpu(), y.cpu(), ly.cpu(), lo.cpu(), sbs), 2e-2, "row panel vs oracle")


@pytest.mark.parametrize("parts_log2,items", [(0, 1), (1, 1), (2, 3), (0, 2), (3, 2)])
def test_row_kernel_parts_and_records_per_workgroup(device, parts_log2, items):
    """The row kernel through the C ABI with rows cut into 1, 2, 4 and 8 column parts and with one, two and
    three records per workgroup (a workgroup then works through consecutive entries of its XCD's list, the
    last workgroups through fewer): the same bits as the tile kernel.  120 block columns: parts of up to 64
    blocks (one mask bit each) and of 15; a work table in reversed order with empty entries.  Every second item
    of a group walks its columns downward (the flag in the table entry), which changes the order of the blocks
    and not the bits."""
    import importlib
    from blksprs_amd import _capi
    from blksprs_amd.utils.tools import build_contraction_lists, pack_layout
    mm = importlib.import_module("blksprs_amd.ops.matmul")
    B, R, K, C, sbs = 2, 5, 6, 120, 64
    if (C + (1 << parts_log2) - 1) >> parts_log2 > 64:
        parts_log2 += 1  # whole rows of 120 blocks do not fit a record: the entry point refuses them (below)
        with pytest.raises(RuntimeError, match="at most 64"):
            _capi.call("bsa_matmul_rows_records", 0, B * R, 0, 8, 8, 8, B * R, C, 0, 8, 0)
    lx, ly = rand_layout((B, R, K), 0.6, seed=1).to(device), rand_layout((B, K, C), 0.5, seed=2).to(device)
    lo = rand_layout((B, R, C), 0.7, seed=3).to(device)
    x = rand_blocks(int(lx.sum()), sbs, torch.bfloat16, 4, 1.0 / math.sqrt(K * sbs)).to(device)
    y = rand_blocks(int(ly.sum()), sbs, torch.bfloat16, 5).to(device)
    info_x, info_y, info_o = pack_layout(lx, row_len=K), pack_layout(ly), pack_layout(lo, row_len=C)
    lists = build_contraction_lists(info_x.packed, info_y.packed, info_o.packed, B, R, K, C, info_o.count)
    table = mm._row_work_table(lists.pair_offsets, info_o.row_offsets, R, parts_log2, pair_up=items == 2,
                               sweep=0 if items == 2 else 1)
    assert items == 2 or int((table >= mm._ROWS_DOWNWARD).sum()) > 0
    table = torch.cat([table.flip(0), torch.full((5,), -1, dtype=torch.int32, device=device)])
    records = mm._row_records(table, parts_log2, lists.pair_offsets, info_x.row_offsets, info_o.row_offsets, B * R, C,
                              info_x.count)
    out = torch.full((info_o.count, sbs, sbs), float("nan"), dtype=torch.bfloat16, device=device)
    _capi.call("bsa_matmul_rows", x.data_ptr(), y.data_ptr(), out.data_ptr(), lists.pair_offsets.data_ptr(),
               _capi.ptr(lists.pairs), records.data_ptr(), records.size(0), items, info_o.count, x.size(0), y.size(0),
               sbs, _capi.BF16, _capi.stream(device))
    ref = torch.empty_like(out)
    _capi.call("bsa_matmul", x.data_ptr(), y.data_ptr(), ref.data_ptr(), lists.pair_offsets.data_ptr(),
               _capi.ptr(lists.pairs), 0, info_o.count, x.size(0), y.size(0), sbs, _capi.BF16, 0, 0,
               _capi.stream(device))
    assert torch.equal(out, ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("trans", ["nn", "grads"])
@pytest.mark.parametrize("dims,density", [
    ((1, 3, 40, 5), 1.0),    # 40 pairs per output block: a run of 8 blocks spans several 64-pair windows
    ((2, 9, 70, 9), 0.95),   # a single output block with more pairs than one window holds
    ((3, 20, 4, 30), 0.3),   # many output blocks without any pair inside a run, runs that end mid-row
    ((1, 1, 1, 1), 1.0),     # one block, one pair: a run shorter than the pipeline is deep
])
def test_sbs16_runs_and_pair_windows(device, dtype, trans, dims, density):
    """The 16-bit sbs-16 kernel hands every wave a run of consecutive output blocks and walks their pairs 64
    at a time with two loads in flight: runs whose pairs cross window boundaries, blocks without pairs, a run
    shorter than the pipeline, and the transposed reads of the backward pass."""
    sbs = 16
    B, R, K, C = dims
    lx, ly, lo, x, y = _problem(B, R, K, C, sbs, dtype, density, seed=R + K, product_layout=density >= 0.9)
    xd, yd = x.to(device).requires_grad_(trans == "grads"), y.to(device).requires_grad_(trans == "grads")
    out = bs.ops.matmul(xd, lx.to(device), yd, ly.to(device), lo.to(device), sbs)
    x64, y64 = x.double().requires_grad_(True), y.double().requires_grad_(True)
    ref = orc.matmul(x64, lx.numpy(), y64, ly.numpy(), lo.numpy(), sbs, acc_dtype=torch.float64)
    assert_close(out, ref, TOL[dtype], f"sbs16 {dtype} {dims}")
    if trans == "grads":
        go = rand_blocks(int(lo.sum()), sbs, dtype, 99, 1.0 / math.sqrt(C * sbs))
        out.backward(go.to(device))
        ref.backward(go.double())
        assert_close(xd.grad, x64.grad, TOL[dtype], "dX")   # x^T-free: go @ y^T reads y transposed
        assert_close(yd.grad, y64.grad, TOL[dtype], "dY")   # x^T @ go reads x transposed


def _tile_kernel_grads(x, y, go, lx, ly, lo, sbs):
    """dX and dY by the tile kernel with transposed operand reads, from contraction lists of the two products."""
    from blksprs_amd import _capi
    from blksprs_amd.utils.tools import build_contraction_lists, pack_layout
    B, R, K = lx.shape
    C = ly.size(2)
    px, py, po = pack_layout(lx), pack_layout(ly), pack_layout(lo)
    pidx_yt = py.packed.view(B, K, C).transpose(1, 2).contiguous().view(-1)
    pidx_xt = px.packed.view(B, R, K).transpose(1, 2).contiguous().view(-1)
    gx, gy = build_contraction_lists((po.packed, pidx_yt, px.packed, B, R, C, K, px.count),
                                     (pidx_xt, po.packed, py.packed, B, K, R, C, py.count))
    dx, dy = torch.empty_like(x), torch.empty_like(y)
    code = _capi.DTYPE_CODES[x.dtype]
    if x.size(0):
        _capi.call("bsa_matmul", go.data_ptr(), y.data_ptr(), dx.data_ptr(), gx.pair_offsets.data_ptr(),
                   _capi.ptr(gx.pairs), 0, x.size(0), go.size(0), y.size(0), sbs, code, 0, 1, _capi.stream(x.device))
    if y.size(0):
        _capi.call("bsa_matmul", x.data_ptr(), go.data_ptr(), dy.data_ptr(), gy.pair_offsets.data_ptr(),
                   _capi.ptr(gy.pairs), 0, y.size(0), x.size(0), go.size(0), sbs, code, 1, 0, _capi.stream(x.device))
    return dx, dy


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dims,dx,dy,do", [
    ((2, 4, 6, 5), 0.5, 0.5, 0.8),      # a few blocks per line: waves without an output block, short lines
    ((2, 3, 40, 70), 0.9, 0.5, 0.9),    # rows of x with more than 16 blocks (several parts), lines of dO of more than 64
    ((1, 70, 20, 3), 0.6, 0.95, 1.0),   # columns of dO of more than 64 blocks, columns of y with more than 16 blocks
    ((3, 9, 7, 11), 0.3, 0.3, 0.5),     # rows without blocks, output blocks without a pair
    ((1, 2, 17, 130), 1.0, 1.0, 1.0),   # dense: 17 output blocks per row (parts of 16 and 1), three segments of dO
])
def test_backward_by_lines_matches_the_tile_kernel_and_the_oracle(device, dtype, dims, dx, dy, do):
    """16-bit operands with 64 x 64 blocks take the line kernel in the backward pass: dX by rows of dO, dY by its
    columns, each line streamed through a ring in LDS that eight waves fill and drain at their own pace.  Held to
    the tile kernel (same products, same order of accumulation inside a block) at the tolerance of the type, to
    autograd of the oracle, and to itself (a second run gives the same bits, whatever the waves' timing)."""
    B, R, K, C = dims
    sbs = 64
    lx = rand_layout((B, R, K), dx, seed=11)
    ly = rand_layout((B, K, C), dy, seed=12)
    lo = rand_layout((B, R, C), do, seed=13)
    if dx < 0.5:
        lx[0, 0] = False
        ly[0, :, 0] = False
    x = rand_blocks(int(lx.sum()), sbs, dtype, 14, 1.0 / math.sqrt(K * sbs))
    y = rand_blocks(int(ly.sum()), sbs, dtype, 15)
    go = rand_blocks(int(lo.sum()), sbs, dtype, 16, 1.0 / math.sqrt(C * sbs))
    lxd, lyd, lod = lx.to(device), ly.to(device), lo.to(device)
    cache = {}
    runs = []
    for _ in range(2):
        xg, yg = x.to(device).requires_grad_(True), y.to(device).requires_grad_(True)
        bs.ops.matmul(xg, lxd, yg, lyd, lod, sbs, layout_cache=cache).backward(go.to(device))
        runs.append((xg.grad, yg.grad))
    assert "grad_x_part_table" in cache and int(cache["grad_lines_error"][0].item()) == 0
    assert torch.equal(runs[0][0], runs[1][0]) and torch.equal(runs[0][1], runs[1][1])
    tile_dx, tile_dy = _tile_kernel_grads(x.to(device), y.to(device), go.to(device), lxd, lyd, lod, sbs)
    assert_close(runs[0][0], tile_dx.double(), 1e-2, "dX by lines against the tile kernel")
    assert_close(runs[0][1], tile_dy.double(), 1e-2, "dY by lines against the tile kernel")
    x64, y64 = x.double().requires_grad_(True), y.double().requires_grad_(True)
    ref = orc.matmul(x64, lx.numpy(), y64, ly.numpy(), lo.numpy(), sbs, acc_dtype=torch.float64)
    ref.backward(go.double())
    assert_close(runs[0][0], x64.grad, 2e-2, "dX by lines against the oracle")
    assert_close(runs[0][1], y64.grad, 2e-2, "dY by lines against the oracle")
    # the part tables, bit for bit: per batch entry first the parts of more than 8 output blocks, then the others,
    # each group in the order of the lines
    def expected_table(counts_per_batch):
        entries = []
        for b, counts in enumerate(counts_per_batch):
            longs, shorts = [], []
            for l, n in enumerate(counts):
                line = b * len(counts) + l
                for p in range((n + 15) // 16):
                    (longs if min(16, n - 16 * p) > 8 else shorts).append(line << 6 | p)
            entries += longs + shorts
        return [len(entries)] + entries

    want_x = expected_table(lx.sum(-1).tolist())
    want_y = expected_table(ly.sum(1).tolist())
    assert cache["grad_x_part_table"].cpu().tolist()[:len(want_x)] == want_x
    assert cache["grad_y_part_table"].cpu().tolist()[:len(want_y)] == want_y


def test_full_size_config2_gradients_sampled_against_the_oracle(device):
    """Config 2 at full size, backward: dX and dY of one batch entry against autograd of the oracle; linearity in
    the upstream gradient (dO -> 2 dO doubles both, bit for bit); a second run gives the same bits."""
    B, n, sbs = 16, 64, 64
    lx = rand_layout((B, n, n), 0.25, seed=0)
    ly = rand_layout((B, n, n), 0.25, seed=1)
    lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
    g = torch.Generator().manual_seed(2)
    x = (torch.randn((int(lx.sum()), sbs, sbs), generator=g) / 64.0).to(torch.bfloat16)
    y = torch.randn((int(ly.sum()), sbs, sbs), generator=g).to(torch.bfloat16)
    go = (torch.randn((int(lo.sum()), sbs, sbs), generator=g) / 64.0).to(torch.bfloat16)
    lxd, lyd, lod = lx.to(device), ly.to(device), lo.to(device)
    cache = {}

    def grads(scale):
        xg, yg = x.to(device).requires_grad_(True), y.to(device).requires_grad_(True)
        bs.ops.matmul(xg, lxd, yg, lyd, lod, sbs, layout_cache=cache).backward(go.to(device) * scale)
        return xg.grad, yg.grad

    dx, dy = grads(1)
    again = grads(1)
    assert torch.equal(dx, again[0]) and torch.equal(dy, again[1])
    doubled = grads(2)
    assert torch.equal(doubled[0], dx * 2) and torch.equal(doubled[1], dy * 2)
    assert int(cache["grad_lines_error"][0].item()) == 0
    b = 5
    sl = lambda lay, t: t[int(lay[:b].sum()):int(lay[:b + 1].sum())]
    x64, y64 = sl(lx, x).double().requires_grad_(True), sl(ly, y).double().requires_grad_(True)
    ref = orc.matmul(x64, lx[b:b + 1].numpy(), y64, ly[b:b + 1].numpy(), lo[b:b + 1].numpy(), sbs,
                     acc_dtype=torch.float64)
    ref.backward(sl(lo, go).double())
    assert_close(sl(lx, dx), x64.grad, 2e-2, "config 2 dX, batch 5")
    assert_close(sl(ly, dy), y64.grad, 2e-2, "config 2 dY, batch 5")


def test_line_kernel_through_the_c_abi_without_an_error_record(device):
    """bsa_matmul_lines_parts + bsa_matmul_lines called directly, with ``error`` NULL (allowed: the bounded waits
    then leave no record) and with part tables built in scratch of exactly the documented size: the same bits as
    the operator's backward pass, for dX and dY; an argument block without output blocks launches nothing."""
    import ctypes
    import sys
    from blksprs_amd import _capi
    mm = sys.modules["blksprs_amd.ops.matmul"]
    B, R, K, C, sbs = 2, 5, 19, 37, 64
    lx, ly, lo = rand_layout((B, R, K), 0.8, seed=41), rand_layout((B, K, C), 0.5, seed=42), rand_layout((B, R, C), 0.7, seed=43)
    x = rand_blocks(int(lx.sum()), sbs, torch.bfloat16, 44, 1.0 / math.sqrt(K * sbs)).to(device)
    y = rand_blocks(int(ly.sum()), sbs, torch.bfloat16, 45).to(device)
    go = rand_blocks(int(lo.sum()), sbs, torch.bfloat16, 46, 1.0 / math.sqrt(C * sbs)).to(device)
    lxd, lyd, lod = lx.to(device), ly.to(device), lo.to(device)
    cache = {}
    xg, yg = x.clone().requires_grad_(True), y.clone().requires_grad_(True)
    bs.ops.matmul(xg, lxd, yg, lyd, lod, sbs, layout_cache=cache).backward(go)
    plan = cache["plan"]
    shapes = ((B, R, K), (B, K, C))
    for which, private, want in (("x", y, xg.grad), ("y", x, yg.grad)):
        out = torch.full(want.shape, float("nan"), dtype=torch.bfloat16, device=device)
        n_lines = B * (R if which == "x" else C)
        scratch = torch.empty(4 * n_lines + 2, dtype=torch.int32, device=device)
        table = torch.full((1 + want.size(0) // 16 + n_lines,), -7, dtype=torch.int32, device=device)
        a = mm._lines_args(plan, shapes, which, go, private, out, table)
        a.error = 0
        _capi.call("bsa_matmul_lines_parts", ctypes.byref(a), scratch.data_ptr(), table.data_ptr(), _capi.stream(device))
        _capi.call("bsa_matmul_lines", ctypes.byref(a), int(which == "y"), sbs, _capi.BF16, _capi.stream(device))
        assert torch.equal(out, want), which
        assert int(table[0]) <= table.numel() - 1
        nothing = mm._lines_args(plan, shapes, which, go, private, None, table)
        nothing.nnz_out, nothing.error = 0, 0
        _capi.call("bsa_matmul_lines", ctypes.byref(nothing), int(which == "y"), sbs, _capi.BF16, _capi.stream(device))
