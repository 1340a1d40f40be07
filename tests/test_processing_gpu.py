"""``bs.utils.apply_torch_linear(_cached)`` and the row-wise callables against the CPU oracle and torch modules.

Modelled on the reference's tests: a linear layer with and without bias on dense and block-sparse inputs, with and
without autocast (test/cases/test_blocksparse.py:1156-1195), the cache of the cached variant
(test/cases/test_regressions.py:535-638), dtype rules (:641-697), empty dimensions (:745-788), normalisation and
dropout through the packed rows (test/cases/test_blocksparse.py:1197-1265) and the argument checks of the row-wise
helper (test/cases/test_regressions.py:2181-2232).

Tolerances: fp32 rtol = atol = 1e-5 on inputs scaled so results are of unit size (fp32 accumulation in another
order than the fp64 oracle); 2e-2 for fp16 / bf16 and under autocast.
"""

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import assert_close, rand_layout

pytestmark = pytest.mark.gpu

SBS = 16


def _linear(in_features, out_features, bias, device, dtype=torch.float32, seed=0):
    torch.manual_seed(seed)
    return torch.nn.Linear(in_features, out_features, bias=bias, device=device, dtype=dtype)


@pytest.mark.parametrize("cached", [False, True])
@pytest.mark.parametrize("use_bias", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sbs,shape,n_out", [(16, (2, 3, 4), 5), (32, (3, 2, 2), 1), (64, (2, 4, 3), 2)])
def test_linear_forward_and_gradients_match_the_oracle(device, cached, use_bias, dtype, sbs, shape, n_out):
    layout = rand_layout(shape, 0.6, seed=sbs + n_out)
    layout[0, 0, :] = 0
    K, N = shape[2] * sbs, n_out * sbs
    g = torch.Generator().manual_seed(sbs)
    x = (torch.randn((int(layout.sum()), sbs, sbs), generator=g) / K ** 0.5).to(dtype)
    linear = _linear(K, N, use_bias, device, dtype, seed=sbs)
    tol = 1e-5 if dtype == torch.float32 else 2e-2

    xd = x.to(device).requires_grad_(True)
    fn = bs.utils.apply_torch_linear_cached if cached else bs.utils.apply_torch_linear
    kwargs = {"layout_cache": {}} if cached else {}
    out, out_layout = fn(bs.BlksprsTensor.wrap(xd), layout.to(device), sbs, linear, **kwargs)
    assert type(out) is bs.BlksprsTensor and out.dtype == dtype
    assert type(out_layout) is torch.Tensor and out_layout.dtype == torch.bool

    xo = x.double().requires_grad_(True)
    wo = linear.weight.detach().cpu().double().requires_grad_(True)
    bo = linear.bias.detach().cpu().double().requires_grad_(True) if use_bias else None
    want, want_layout = orc.linear(xo, layout.numpy(), wo, bo, sbs)
    assert torch.equal(out_layout.cpu(), torch.as_tensor(want_layout))
    assert_close(out, want, tol, "output")

    grad = torch.randn(want.shape, generator=g, dtype=torch.float64)
    want.backward(grad)
    out.backward(grad.to(device=device, dtype=dtype))
    gtol = tol * 4
    assert_close(xd.grad, xo.grad, gtol, "grad x")
    assert_close(linear.weight.grad, wo.grad, gtol * max(1.0, float(wo.grad.abs().max())), "grad weight")
    if use_bias:
        assert_close(linear.bias.grad, bo.grad, gtol * max(1.0, float(bo.grad.abs().max())), "grad bias")


@pytest.mark.parametrize("cached", [False, True])
@pytest.mark.parametrize("use_bias", [False, True])
def test_linear_matches_torch_on_dense_and_sparse_inputs_under_autocast(device, cached, use_bias):
    """test/cases/test_blocksparse.py:1156-1184 at one configuration, autocast on and off."""
    b, m, k, n, sbs = 2, 64, 96, 32, 32
    g = torch.Generator().manual_seed(4)
    dense = torch.randn((b, m, k), generator=g).to(device)
    sparse_layout = rand_layout((b, m // sbs, k // sbs), 0.5, seed=5).to(device)
    keep = sparse_layout.repeat_interleave(sbs, 1).repeat_interleave(sbs, 2) != 0
    linear = _linear(k, n, use_bias, device)
    fn = bs.utils.apply_torch_linear_cached if cached else bs.utils.apply_torch_linear
    for use_amp in (False, True):
        with torch.amp.autocast(device_type="cuda", enabled=use_amp):
            for x, layout in ((dense, torch.ones_like(sparse_layout)), (dense * keep, sparse_layout)):
                want = linear(x)
                kwargs = {"layout_cache": {}} if cached else {}
                out, out_layout = fn(bs.ops.to_sparse(x, layout, sbs), layout, sbs, linear, **kwargs)
                got = bs.ops.to_dense(out, out_layout, sbs)
                assert out.dtype == want.dtype
                if not use_bias:  # rows without input blocks give zeros in both
                    want = want * (out_layout.repeat_interleave(sbs, 1).repeat_interleave(sbs, 2) != 0)
                assert_close(got.float(), want.float(), 2e-2 if use_amp else 1e-4, f"amp={use_amp}")


def test_linear_rejects_bad_arguments(device):
    """test/cases/test_blocksparse.py:1187-1195, test/cases/test_regressions.py:641-662."""
    layout = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    x = bs.BlksprsTensor.wrap(torch.zeros((1, SBS, SBS), device=device))
    with pytest.raises(ValueError, match="divisible"):
        bs.utils.apply_torch_linear(x, layout, SBS, _linear(SBS + 1, SBS, False, device))
    with pytest.raises(ValueError, match="divisible"):
        bs.utils.apply_torch_linear(x, layout, SBS, _linear(SBS, SBS + 1, True, device))
    half = bs.BlksprsTensor.wrap(x.half())
    for fn, kwargs in ((bs.utils.apply_torch_linear, {}), (bs.utils.apply_torch_linear_cached, {"layout_cache": {}})):
        with pytest.raises(ValueError, match="same dtype"):
            fn(half, layout, SBS, _linear(SBS, SBS, True, device), **kwargs)


@pytest.mark.parametrize("cached", [False, True])
def test_linear_bias_keeps_the_autocast_dtype_and_all_gradients(device, cached):
    """test/cases/test_regressions.py:665-697."""
    layout = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    linear = _linear(SBS, SBS, True, device)
    cache = {}
    for _ in range(2):
        dense = torch.randn((1, SBS, SBS), device=device, requires_grad=True)
        sparse = bs.ops.to_sparse(dense, layout, SBS)
        with torch.amp.autocast(device_type="cuda", dtype=torch.float16):
            expected = linear(dense)
            if cached:
                actual, actual_layout = bs.utils.apply_torch_linear_cached(sparse, layout, SBS, linear,
                                                                           layout_cache=cache)
            else:
                actual, actual_layout = bs.utils.apply_torch_linear(sparse, layout, SBS, linear)
            actual_dense = bs.ops.to_dense(actual, actual_layout, SBS)
        gradient = torch.randn_like(expected)
        inputs = (dense, linear.weight, linear.bias)
        expected_gradients = torch.autograd.grad(expected, inputs, gradient, retain_graph=True)
        actual_gradients = torch.autograd.grad(actual_dense, inputs, gradient)
        assert actual.dtype == expected.dtype
        assert torch.allclose(actual_dense, expected, atol=2e-2, rtol=1e-2)
        for a, e in zip(actual_gradients, expected_gradients):
            assert torch.allclose(a, e, atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize("cached", [False, True])
@pytest.mark.parametrize("batch,row_blocks,in_features", [(1, 2, 0), (1, 0, SBS), (0, 2, SBS)])
def test_linear_bias_on_empty_dimensions(device, cached, batch, row_blocks, in_features):
    """test/cases/test_regressions.py:745-788."""
    layout = torch.ones((batch, row_blocks, in_features // SBS), dtype=torch.bool, device=device)
    dense = torch.empty((batch, row_blocks * SBS, in_features), device=device, requires_grad=True)
    sparse = bs.ops.to_sparse(dense, layout, SBS)
    linear = _linear(in_features, SBS, True, device)
    expected = linear(dense)
    if cached:
        actual, actual_layout = bs.utils.apply_torch_linear_cached(sparse, layout, SBS, linear, layout_cache={})
    else:
        actual, actual_layout = bs.utils.apply_torch_linear(sparse, layout, SBS, linear)
    actual_dense = bs.ops.to_dense(actual, actual_layout, SBS)
    gradient = torch.randn_like(expected)
    inputs = (dense, linear.weight, linear.bias)
    expected_gradients = torch.autograd.grad(expected, inputs, gradient, retain_graph=True)
    actual_gradients = torch.autograd.grad(actual_dense, inputs, gradient)
    assert type(actual_layout) is torch.Tensor
    assert actual_layout.shape == (batch, row_blocks, 1) and torch.all(actual_layout)
    assert torch.allclose(actual_dense, expected)
    for a, e in zip(actual_gradients, expected_gradients):
        assert torch.allclose(a, e)


def test_linear_cache_follows_layout_and_parameter_state(device):
    """test/cases/test_regressions.py:535-638."""
    first = torch.tensor([[[True], [False]]], device=device)
    second = torch.tensor([[[False], [True]]], device=device)
    linear = _linear(SBS, SBS, False, device)
    cache = {}
    dense = torch.zeros((1, SBS * 2, SBS), device=device)
    dense[:, :SBS] = 1
    bs.utils.apply_torch_linear_cached(bs.ops.to_sparse(dense, first, SBS), first, SBS, linear, layout_cache=cache)
    dense.fill_(0)
    dense[:, SBS:] = 2
    sparse = bs.ops.to_sparse(dense, second, SBS)
    actual, actual_layout = bs.utils.apply_torch_linear_cached(sparse, second, SBS, linear, layout_cache=cache)
    expected, expected_layout = bs.utils.apply_torch_linear_cached(sparse, second, SBS, linear, layout_cache={})
    assert torch.equal(actual_layout, expected_layout) and torch.allclose(actual, expected)

    # a hit keeps the compressed parameters, a change of requires_grad or of the gradient mode replaces them
    layout = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    dense = torch.randn((1, SBS, SBS), device=device, requires_grad=True)
    sparse = bs.ops.to_sparse(dense, layout, SBS)
    linear = _linear(SBS, SBS, True, device)
    cache = {}
    with torch.no_grad():
        bs.utils.apply_torch_linear_cached(sparse, layout, SBS, linear, layout_cache=cache)
    evaluation_weight, evaluation_bias = cache["w_t_bs"], cache["bias_slice_bs"]
    output, _ = bs.utils.apply_torch_linear_cached(sparse, layout, SBS, linear, layout_cache=cache)
    assert cache["w_t_bs"] is not evaluation_weight and cache["w_t_bs"].requires_grad
    assert cache["bias_slice_bs"] is not evaluation_bias and cache["bias_slice_bs"].requires_grad
    training_weight = cache["w_t_bs"]
    output2, _ = bs.utils.apply_torch_linear_cached(sparse, layout, SBS, linear, layout_cache=cache)
    assert cache["w_t_bs"] is training_weight and torch.equal(output, output2)
    (output + output2).sum().backward()
    assert dense.grad is not None and linear.weight.grad is not None and linear.bias.grad is not None
    linear.weight.requires_grad_(False)
    linear.weight.grad = None
    output3, _ = bs.utils.apply_torch_linear_cached(sparse, layout, SBS, linear, layout_cache=cache)
    assert cache["w_t_bs"] is not training_weight and not cache["w_t_bs"].requires_grad
    output3.sum().backward()
    assert linear.weight.grad is None


def test_linear_cache_survives_training_iterations(device):
    """Forward and backward, three times over: the compressed parameters and the product's lookup tables are
    built once (the lists the backward pass adds to the product's cache do not invalidate the linear cache)."""
    layout = rand_layout((2, 3, 2), 0.7, seed=3).to(device)
    linear = _linear(2 * SBS, 3 * SBS, True, device)
    dense = torch.randn((2, 3 * SBS, 2 * SBS), device=device)
    sparse = bs.ops.to_sparse(dense, layout, SBS)
    cache = {}
    seen = []
    for _ in range(3):
        out, _ = bs.utils.apply_torch_linear_cached(sparse, layout, SBS, linear, layout_cache=cache)
        out.square().sum().backward()
        product_cache = cache["matmul_layout_cache"].cache
        seen.append((cache["w_t_bs"], product_cache["contraction_pairs"], product_cache["grad_x_pairs"]))
        linear.zero_grad(set_to_none=False)  # in place: the parameters stay the same objects and versions...
    # ... except that zeroing bumps the version of .grad only, not of the parameters
    assert all(a is b for a, b in zip(seen[0], seen[1])) and all(a is b for a, b in zip(seen[1], seen[2]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_normalisation_and_dropout_through_packed_rows(device, dtype):
    """test/cases/test_blocksparse.py:1197-1265: layer norm over the feature dimension of a tensor whose inactive
    blocks are zero equals the module on the dense tensor, on the active blocks; dropout in eval mode is the
    identity and in training mode zeroes or rescales every element."""
    sbs, shape = 32, (2, 3, 4)
    layout = rand_layout(shape, 0.6, seed=8)
    layout[1, 1, :] = 0
    g = torch.Generator().manual_seed(9)
    dense = torch.randn((2, 3 * sbs, 4 * sbs), generator=g).to(dtype)
    x = orc.to_sparse(dense, layout.numpy(), sbs)
    xd, ld = bs.BlksprsTensor.wrap(x.to(device)), layout.to(device)
    norm = torch.nn.LayerNorm(4 * sbs, device=device, dtype=dtype)
    got = bs.utils.apply_torch_normalisation(xd, ld, sbs, norm)
    assert type(got) is bs.BlksprsTensor and got.shape == x.shape
    masked = orc.to_dense(x, layout.numpy(), sbs)
    want = orc.to_sparse(torch.nn.functional.layer_norm(masked.double(), (4 * sbs,)), layout.numpy(), sbs)
    assert_close(got, want, 1e-5 if dtype == torch.float32 else 2e-2, "layer norm")
    drop = torch.nn.Dropout(0.5).eval()
    assert torch.equal(bs.utils.apply_torch_dropout(xd, ld, sbs, drop).cpu(), x)
    dropped = bs.utils.apply_torch_dropout(xd, ld, sbs, drop.train()).cpu()
    assert torch.all((dropped == 0) | (dropped == x * 2))
    assert 0.3 < float((dropped == 0).float().mean()) < 0.7


def test_row_wise_helper_checks_its_arguments(device):
    """test/cases/test_regressions.py:2181-2232."""
    layout = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    x = bs.BlksprsTensor.wrap(torch.randn((1, SBS, SBS), device=device))
    with pytest.raises(ValueError):
        bs.utils.apply_function_applicable_row_wise(
            bs.BlksprsTensor.wrap(torch.randn((2, SBS, SBS), device=device)), layout, SBS, lambda t: t)
    with pytest.raises(TypeError, match="must be callable"):
        bs.utils.apply_function_applicable_row_wise(x, layout, SBS, None)
    with pytest.raises(TypeError, match="must return a Tensor"):
        bs.utils.apply_function_applicable_row_wise(x, layout, SBS, lambda t: None)
    with pytest.raises(ValueError, match="shape"):
        bs.utils.apply_function_applicable_row_wise(x, layout, SBS, lambda t: t[..., :1])
    with pytest.raises(ValueError, match="GPU|device"):
        bs.utils.apply_function_applicable_row_wise(x, layout, SBS, lambda t: t.cpu())
    out = bs.utils.apply_function_applicable_row_wise(x, layout, SBS, lambda t: t.to(torch.float64))
    assert out.dtype == torch.float64 and torch.equal(out.float(), x)
    empty = torch.zeros((2, 2, 2), dtype=torch.bool, device=device)
    nothing = bs.BlksprsTensor.wrap(torch.empty((0, SBS, SBS), device=device))
    assert bs.utils.apply_function_applicable_row_wise(nothing, empty, SBS, lambda t: t).shape == (0, SBS, SBS)


def test_product_layout_approximations(device):
    """fast = rows AND columns, outer = rows OR columns (blksprs/layouting/sparsity_layout.py:262-311); the exact
    product lies inside the fast one; empty inner dimensions give an empty fast layout
    (test/cases/test_regressions.py:1200-1215)."""
    lx = rand_layout((3, 4, 5), 0.3, seed=1)
    ly = rand_layout((3, 5, 6), 0.3, seed=2)
    rows, cols = lx.any(-1, keepdim=True), ly.any(-2, keepdim=True)
    fast = bs.layouting.build_sparsity_layout_matmul_fast(lx.to(device), ly.to(device))
    outer = bs.layouting.build_sparsity_layout_matmul_outer(lx.to(device), ly.to(device))
    exact = bs.layouting.build_sparsity_layout_matmul(lx.to(device), ly.to(device))
    assert type(fast) is torch.Tensor and fast.dtype == torch.bool
    assert torch.equal(fast.cpu(), rows & cols) and torch.equal(outer.cpu(), rows | cols)
    assert torch.all(fast | ~exact) and torch.all(outer | ~fast)
    left = torch.empty((1, 2, 0), dtype=torch.bool, device=device)
    right = torch.empty((1, 0, 3), dtype=torch.bool, device=device)
    for builder in (bs.layouting.build_sparsity_layout_matmul_fast, bs.layouting.build_sparsity_layout_matmul_outer):
        out = builder(left, right)
        assert out.shape == (1, 2, 3) and not torch.any(out)
    with pytest.raises(ValueError, match="Inner dimensions"):
        bs.layouting.build_sparsity_layout_matmul_fast(lx.to(device), lx.to(device))
