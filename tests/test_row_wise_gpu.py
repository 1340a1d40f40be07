"""Parity of ``bs.ops.misc.row_wise_sum / row_wise_max / row_wise_add / row_wise_sub`` with the CPU oracle.

Modelled on the reference's tests: sums, maxima and the add of the maxima against dense torch through a
conversion round trip (test/cases/test_blocksparse.py:789-886), fp32 accumulation of a bf16 sum
(test/cases/test_regressions.py:132-146), dtype, -inf and NaN behaviour of the maximum (:1162-1183,
:1981-2004), empty logical columns (:1218-1236, :1298-1310), slices as auxiliary plain tensors (:1239-1256),
mixed dtypes rejected (:1286-1295), returned layouts are plain tensors (:1696-1712).

Tolerances: the maximum and the add of an exactly representable value are exact; sums accumulate in fp32 in
another order than the fp64 oracle, so fp32 results are held to rtol = atol = 1e-5 on inputs of unit scale and
16-bit results to one rounding of the storage type (2e-2).
"""

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import rand_layout

pytestmark = pytest.mark.gpu

FLOATS = [torch.float16, torch.bfloat16, torch.float32]
TOL = {torch.float32: 1e-5, torch.float16: 2e-2, torch.bfloat16: 2e-2}
SHAPES = [(16, (2, 3, 5)), (32, (3, 4, 2)), (64, (2, 5, 7)), (128, (1, 2, 3)), (256, (1, 2, 2))]


def _case(sbs, shape, dtype, seed, density=0.6):
    layout = rand_layout(shape, density, seed=seed)
    layout[0, 0, :] = 0  # a block row without blocks
    if shape[1] > 1:
        layout[-1, -1, :] = 1  # and a full one
    g = torch.Generator().manual_seed(seed + 1)
    x = torch.randn((int(layout.sum()), sbs, sbs), generator=g).to(dtype)
    return layout, x


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("sbs,shape", SHAPES)
@pytest.mark.parametrize("slice_only", [False, True])
def test_row_wise_sum(device, dtype, sbs, shape, slice_only):
    layout, x = _case(sbs, shape, dtype, seed=sbs)
    out, out_layout = bs.ops.misc.row_wise_sum(bs.BlksprsTensor.wrap(x.to(device)), layout.to(device), sbs,
                                               flag_slice_only=slice_only)
    want, want_layout = orc.row_wise_reduce(x, layout.numpy(), sbs, "sum", slice_only)
    assert out.dtype == dtype and out.shape == want.shape
    assert type(out) is (torch.Tensor if slice_only else bs.BlksprsTensor)
    assert type(out_layout) is torch.Tensor and out_layout.shape == (shape[0], shape[1], 1)
    assert torch.equal(out_layout.cpu() != 0, torch.as_tensor(want_layout))
    torch.testing.assert_close(out.cpu().float(), want.float(), rtol=TOL[dtype], atol=TOL[dtype] * 8)
    if not slice_only:
        assert torch.all(out[..., 1:] == 0)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("sbs,shape", SHAPES)
@pytest.mark.parametrize("slice_only", [False, True])
def test_row_wise_max_is_exact(device, dtype, sbs, shape, slice_only):
    layout, x = _case(sbs, shape, dtype, seed=sbs + 3)
    x[0, 1, :] = float("-inf")
    x[-1, 2, 5] = float("nan")
    out, out_layout = bs.ops.misc.row_wise_max(bs.BlksprsTensor.wrap(x.to(device)), layout.to(device), sbs,
                                               flag_slice_only=slice_only)
    want, want_layout = orc.row_wise_reduce(x, layout.numpy(), sbs, "max", slice_only)
    assert out.dtype == dtype and out.shape == want.shape
    assert torch.equal(out_layout.cpu() != 0, torch.as_tensor(want_layout))
    got = out.cpu()
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    assert torch.isnan(want).any()
    assert torch.equal(torch.nan_to_num(got, nan=0.0), torch.nan_to_num(want, nan=0.0))
    if not slice_only:
        assert torch.all(torch.isneginf(out[..., 1:]))


@pytest.mark.parametrize("dtype,sbs", [(torch.float32, 512), (torch.bfloat16, 1024)])
def test_rows_wider_than_one_wave(device, dtype, sbs):
    """More than 64 vectors of 16 bytes per element row: a lane then holds several vectors of a row."""
    layout = torch.tensor([[[1, 0, 1]]])
    g = torch.Generator().manual_seed(sbs)
    x = torch.randn((2, sbs, sbs), generator=g).to(dtype)
    xd, ld = bs.BlksprsTensor.wrap(x.to(device)), layout.to(device)
    for op, name in ((bs.ops.misc.row_wise_sum, "sum"), (bs.ops.misc.row_wise_max, "max")):
        for slice_only in (False, True):
            out, _ = op(xd, ld, sbs, flag_slice_only=slice_only)
            want, _ = orc.row_wise_reduce(x, layout.numpy(), sbs, name, slice_only)
            torch.testing.assert_close(out.cpu().float(), want.float(), rtol=TOL[dtype], atol=TOL[dtype] * 32)
    vals, _ = bs.ops.misc.row_wise_max(xd, ld, sbs, flag_slice_only=True)
    got = bs.ops.misc.row_wise_sub(xd, ld, vals, sbs)
    want = orc.row_wise_add(x, layout.numpy(), -vals.cpu(), sbs)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("sbs,shape", SHAPES)
@pytest.mark.parametrize("y_square", [False, True])
def test_row_wise_add_and_sub(device, dtype, sbs, shape, y_square):
    layout, x = _case(sbs, shape, dtype, seed=sbs + 9)
    n_rows = int((layout.sum(-1) > 0).sum())
    g = torch.Generator().manual_seed(sbs + 10)
    y = torch.randn((n_rows, sbs, sbs if y_square else 1), generator=g).to(dtype)
    xd, ld = bs.BlksprsTensor.wrap(x.to(device)), layout.to(device)
    got = bs.ops.misc.row_wise_add(xd, ld, y.to(device), sbs)
    assert type(got) is bs.BlksprsTensor and got.dtype == dtype and got.shape == x.shape
    # one rounding of the exact sum of two storage-type values: bit-exact against the fp64 oracle
    assert torch.equal(got.cpu(), orc.row_wise_add(x, layout.numpy(), y, sbs))
    got = bs.ops.misc.row_wise_sub(xd, ld, y.to(device), sbs)
    assert torch.equal(got.cpu(), orc.row_wise_add(x, layout.numpy(), -y, sbs))


@pytest.mark.parametrize("dtype", FLOATS)
def test_softmax_from_its_parts(device, dtype):
    """exp(x - max) / sum(exp(x - max)) built from the row-wise operations equals the dense softmax
    (the composition the reference's regular softmax is made of, blksprs/ops/softmax.py:93-144)."""
    sbs = 32
    layout = rand_layout((2, 4, 6), 0.5, seed=77, ensure_rows=True)
    g = torch.Generator().manual_seed(78)
    x = torch.randn((int(layout.sum()), sbs, sbs), generator=g).to(dtype)
    xd, ld = bs.BlksprsTensor.wrap(x.to(device)), layout.to(device)
    row_max, _ = bs.ops.misc.row_wise_max(xd, ld, sbs, flag_slice_only=True)
    shifted = torch.exp(bs.ops.misc.row_wise_sub(xd, ld, row_max, sbs))
    total, _ = bs.ops.misc.row_wise_sum(bs.BlksprsTensor.wrap(shifted), ld, sbs, flag_slice_only=True)
    out = shifted / total.repeat_interleave((layout.sum(-1)[layout.sum(-1) > 0]).to(device), dim=0)
    want = orc.softmax(x.double(), layout.numpy(), sbs)
    torch.testing.assert_close(out.cpu().double(), want, rtol=TOL[dtype], atol=TOL[dtype])


def test_sum_of_bf16_ones_accumulates_in_fp32(device):
    """test/cases/test_regressions.py:132-146: 16384 ones in bf16 sum to exactly 16384."""
    sbs, columns = 16, 16_384
    n = columns // sbs
    layout = torch.ones((1, 1, n), dtype=torch.bool, device=device)
    x = bs.BlksprsTensor.wrap(torch.ones((n, sbs, sbs), dtype=torch.bfloat16, device=device))
    out, out_layout = bs.ops.misc.row_wise_sum(x, layout, sbs, flag_slice_only=True)
    assert out.dtype == torch.bfloat16 and out_layout.shape == (1, 1, 1)
    assert torch.all(out == columns)


@pytest.mark.parametrize("dtype", FLOATS)
def test_max_keeps_dtype_negative_infinity_and_nan_of_any_block(device, dtype):
    """test/cases/test_regressions.py:1162-1183, :1981-2004."""
    sbs = 16
    full = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    x = bs.BlksprsTensor.wrap(torch.full((1, sbs, sbs), float("-inf"), dtype=dtype, device=device))
    out, _ = bs.ops.misc.row_wise_max(x, full, sbs)
    assert out.dtype == dtype and torch.all(torch.isneginf(out))
    two = torch.ones((1, 1, 2), dtype=torch.bool, device=device)
    dense = torch.arange(sbs * sbs * 2, dtype=torch.float32, device=device).reshape(1, sbs, sbs * 2).to(dtype)
    dense[0, 0, 0] = float("nan")
    dense[0, 1, sbs] = float("nan")
    out, out_layout = bs.ops.misc.row_wise_max(bs.ops.to_sparse(dense, two, sbs), two, sbs)
    actual = bs.ops.to_dense(out, out_layout, sbs)[..., 0]
    expected = torch.max(dense, dim=-1).values
    assert out.dtype == dtype
    assert torch.equal(torch.isnan(actual), torch.isnan(expected))
    assert torch.equal(torch.nan_to_num(actual, nan=0.0), torch.nan_to_num(expected, nan=0.0))


@pytest.mark.parametrize("op", ["sum", "max"])
@pytest.mark.parametrize("slice_only", [False, True])
@pytest.mark.parametrize("shape", [(1, 2, 0), (0, 1, 1), (1, 0, 1), (1, 2, 3)])
def test_reductions_accept_empty_inputs(device, op, slice_only, shape):
    """test/cases/test_regressions.py:1218-1236 (and layouts without any block)."""
    sbs = 16
    fn = bs.ops.misc.row_wise_sum if op == "sum" else bs.ops.misc.row_wise_max
    layout = torch.zeros(shape, dtype=torch.bool, device=device)
    x = bs.BlksprsTensor.wrap(torch.empty((0, sbs, sbs), device=device))
    out, out_layout = fn(x, layout, sbs, flag_slice_only=slice_only)
    assert type(out) is (torch.Tensor if slice_only else bs.BlksprsTensor)
    assert out.shape == (0, sbs, 1 if slice_only else sbs)
    assert out_layout.shape == (shape[0], shape[1], 1) and not torch.any(out_layout)


@pytest.mark.parametrize("op", ["add", "sub"])
@pytest.mark.parametrize("shape", [(1, 2, 0), (0, 1, 1), (1, 0, 1), (1, 2, 3)])
def test_arithmetic_accepts_empty_inputs(device, op, shape):
    """test/cases/test_regressions.py:1298-1310."""
    sbs = 16
    fn = bs.ops.misc.row_wise_add if op == "add" else bs.ops.misc.row_wise_sub
    layout = torch.zeros(shape, dtype=torch.bool, device=device)
    x = bs.BlksprsTensor.wrap(torch.empty((0, sbs, sbs), device=device))
    y = torch.empty((0, sbs, 1), device=device)
    out = fn(x, layout, y, sbs)
    assert type(out) is bs.BlksprsTensor and out.shape == x.shape


def test_slices_feed_the_arithmetic_and_errors(device):
    """test/cases/test_regressions.py:1239-1256, :1286-1295, and the two conformity errors of
    blksprs/ops/misc/row_wise.py:456-461."""
    sbs = 16
    layout = torch.ones((1, 1, 2), dtype=torch.bool, device=device)
    x = bs.BlksprsTensor.wrap(torch.randn((2, sbs, sbs), device=device))
    for fn in (bs.ops.misc.row_wise_sum, bs.ops.misc.row_wise_max):
        out, out_layout = fn(x, bs.BlksprsTensor.wrap(layout), sbs, flag_slice_only=True)
        assert type(out) is torch.Tensor and out.shape == (1, sbs, 1)
        assert type(out_layout) is torch.Tensor and out_layout.shape == (1, 1, 1)
        assert type(bs.ops.misc.row_wise_add(x, layout, out, sbs)) is bs.BlksprsTensor
    with pytest.raises(ValueError, match="same dtype"):
        bs.ops.misc.row_wise_add(bs.BlksprsTensor.wrap(x.half()), layout, torch.randn((1, sbs, 1), device=device), sbs)
    with pytest.raises(ValueError, match="does not conform"):
        bs.ops.misc.row_wise_add(x, layout, torch.randn((2, sbs, 1), device=device), sbs)
    with pytest.raises(ValueError, match="either 1 or sparsity block size columns"):
        bs.ops.misc.row_wise_add(x, layout, torch.randn((1, sbs, 2), device=device), sbs)
    with pytest.raises(ValueError, match="float16, bfloat16, or float32"):
        bs.ops.misc.row_wise_sum(bs.BlksprsTensor.wrap(x.double()), layout, sbs)


def test_results_carry_no_gradient(device):
    sbs = 16
    layout = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    x = torch.randn((1, sbs, sbs), device=device, requires_grad=True)
    out, _ = bs.ops.misc.row_wise_sum(bs.BlksprsTensor.wrap(x), layout, sbs)
    assert not out.requires_grad
    assert not bs.ops.misc.row_wise_add(bs.BlksprsTensor.wrap(x), layout, out, sbs).requires_grad
