"""Edge cases the reference pins in test/cases/test_regressions.py and test/cases/test_readme.py, restated against
dense torch on the same inputs, plus the sequences in which one layout cache serves several calls between a forward
and its backward pass."""

import math

import pytest
import torch

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import assert_close, rand_blocks, rand_layout

pytestmark = pytest.mark.gpu

# (dtype, block size): the matrix-core attention kernels (16-bit, 64) and the generic ones
ATTENTION_PATHS = [(torch.bfloat16, 64), (torch.float16, 64), (torch.float32, 16), (torch.float32, 64)]


def _full(device, rows=1, cols=1):
    return torch.ones((1, rows, cols), dtype=torch.bool, device=device)


def _simple_attention(q, k, v, sbs, scale=None, bias=None):
    lay = _full(q.device)
    return bs.ops.flash_attention(q, lay, k, lay, v, lay, lay, sbs, scale=scale, attention_bias=bias,
                                  sparsity_layout_bias=None if bias is None else lay, sparsity_layout_o=lay)


@pytest.mark.parametrize("dtype,sbs", ATTENTION_PATHS)
@pytest.mark.parametrize("where", ["q", "k", "bias"])
def test_attention_propagates_non_finite_inputs(device, dtype, sbs, where):
    """test/cases/test_regressions.py:2007-2033: a NaN in q, k or the bias shows up in the output exactly where it
    does in ``softmax(q k^T / sqrt(d) + bias) v`` on the dense tensors."""
    q, k, v = (rand_blocks(1, sbs, dtype, s).to(device) for s in (1, 2, 3))
    bias = torch.zeros_like(q) if where == "bias" else None
    {"q": q, "k": k, "bias": bias}[where][0, 0, 0] = float("nan")
    actual = _simple_attention(q, k, v, sbs, bias=bias)
    scores = torch.bmm(q.float(), k.float().transpose(-2, -1)) / sbs ** 0.5
    if bias is not None:
        scores = scores + bias.float()
    expected = torch.bmm(torch.softmax(scores, dim=-1), v.float())
    assert torch.equal(torch.isnan(actual), torch.isnan(expected))
    assert torch.isnan(actual).any()


@pytest.mark.parametrize("dtype,sbs", ATTENTION_PATHS)
@pytest.mark.parametrize("scale", [float("nan"), float("inf")])
def test_attention_propagates_non_finite_scale(device, dtype, sbs, scale):
    """test/cases/test_regressions.py:2036-2049: a NaN or infinite scale makes every output NaN, as it does in
    dense torch (inf - inf in the softmax)."""
    q = torch.ones((1, sbs, sbs), dtype=dtype, device=device)
    k = torch.ones_like(q)
    v = rand_blocks(1, sbs, dtype, 3).to(device)
    actual = _simple_attention(q, k, v, sbs, scale=scale)
    scores = torch.bmm(q.float(), k.float().transpose(-2, -1)) * scale
    expected = torch.bmm(torch.softmax(scores, dim=-1), v.float())
    assert torch.equal(torch.isnan(actual), torch.isnan(expected))
    assert torch.isnan(actual).any()


@pytest.mark.parametrize("dtype,sbs", ATTENTION_PATHS)
def test_attention_backward_propagates_nan_bias(device, dtype, sbs):
    """test/cases/test_regressions.py:2052-2076: a NaN in the bias reaches every gradient."""
    lay = _full(device)
    q, k, v = (rand_blocks(1, sbs, dtype, s).to(device).requires_grad_(True) for s in (1, 2, 3))
    bias = torch.zeros((1, sbs, sbs), dtype=dtype, device=device)
    bias[0, 0, 0] = float("nan")
    bias.requires_grad_(True)
    out = bs.ops.flash_attention(q, lay, k, lay, v, lay, lay, sbs, attention_bias=bias, sparsity_layout_bias=lay,
                                 sparsity_layout_o=lay)
    grads = torch.autograd.grad(out.float().sum(), (q, k, v, bias))
    assert all(torch.isnan(g).any() for g in grads)


def _non_contiguous(n, sbs, dtype, device, seed):
    g = torch.Generator().manual_seed(seed)
    base = torch.randn((n, sbs, 2 * sbs), generator=g).to(dtype).to(device)
    grad = base[:, :, ::2]
    assert not grad.is_contiguous()
    return grad


@pytest.mark.parametrize("dtype,sbs", ATTENTION_PATHS)
def test_attention_backward_takes_a_non_contiguous_output_gradient(device, dtype, sbs):
    """test/cases/test_regressions.py:279-315: same gradients as with the contiguous copy."""
    lay = _full(device)
    values = [rand_blocks(1, sbs, dtype, s).to(device) for s in (1, 2, 3)]
    grad = _non_contiguous(1, sbs, dtype, device, 4)
    results = []
    for g in (grad, grad.contiguous()):
        inputs = [t.clone().requires_grad_(True) for t in values]
        out = bs.ops.flash_attention(inputs[0], lay, inputs[1], lay, inputs[2], lay, lay, sbs)
        results.append(torch.autograd.grad(out, inputs, g))
    for a, b in zip(*results):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype,sbs", [(torch.bfloat16, 64), (torch.float32, 32), (torch.float16, 16)])
def test_matmul_backward_takes_a_non_contiguous_output_gradient(device, dtype, sbs):
    lx, ly = rand_layout((2, 3, 4), 0.6, 1, ensure_rows=True), rand_layout((2, 4, 3), 0.6, 2, ensure_rows=True)
    lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
    x, y = rand_blocks(int(lx.sum()), sbs, dtype, 3).to(device), rand_blocks(int(ly.sum()), sbs, dtype, 4).to(device)
    grad = _non_contiguous(int(lo.sum()), sbs, dtype, device, 5)
    results = []
    for g in (grad, grad.contiguous()):
        xs, ys = x.clone().requires_grad_(True), y.clone().requires_grad_(True)
        out = bs.ops.matmul(xs, lx.to(device), ys, ly.to(device), lo.to(device), sbs)
        results.append(torch.autograd.grad(out, (xs, ys), g))
    for a, b in zip(*results):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype,sbs", [(torch.bfloat16, 64), (torch.float32, 32)])
def test_matmul_backward_after_the_cache_served_other_layouts(device, dtype, sbs):
    """Two products with different layouts through ONE cache dict, then the backward pass of both: each uses the
    lists of its own forward pass (the second call empties and refills the dict).  Compared with separate caches."""
    def problem(seed, dims):
        B, R, K, C = dims
        lx, ly = rand_layout((B, R, K), 0.6, seed, ensure_rows=True), rand_layout((B, K, C), 0.6, seed + 1, ensure_rows=True)
        lo = torch.from_numpy(orc.layout_matmul(lx.numpy(), ly.numpy()))
        x, y = rand_blocks(int(lx.sum()), sbs, dtype, seed + 2), rand_blocks(int(ly.sum()), sbs, dtype, seed + 3)
        go = rand_blocks(int(lo.sum()), sbs, dtype, seed + 4, 1.0 / math.sqrt(K * sbs))
        return [t.to(device) for t in (lx, ly, lo, x, y, go)]

    # the first has more x blocks than the second and equal layout shapes; the third differs in shape
    problems = [problem(10, (2, 5, 6, 4)), problem(20, (2, 5, 6, 4)), problem(30, (1, 3, 2, 5))]
    expected = []
    for lx, ly, lo, x, y, go in problems:
        xs, ys = x.clone().requires_grad_(True), y.clone().requires_grad_(True)
        expected.append(torch.autograd.grad(bs.ops.matmul(xs, lx, ys, ly, lo, sbs, layout_cache={}), (xs, ys), go))
    shared, outs, leaves = {}, [], []
    for lx, ly, lo, x, y, go in problems:
        xs, ys = x.clone().requires_grad_(True), y.clone().requires_grad_(True)
        outs.append(bs.ops.matmul(xs, lx, ys, ly, lo, sbs, layout_cache=shared))
        leaves.append((xs, ys))
    for out, (xs, ys), (_, _, _, _, _, go), want in zip(outs, leaves, problems, expected):
        got = torch.autograd.grad(out, (xs, ys), go)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


@pytest.mark.parametrize("dtype,sbs", [(torch.bfloat16, 64), (torch.float32, 16)])
def test_attention_backward_after_the_cache_served_other_layouts(device, dtype, sbs):
    """As above for attention, with a mask: the second and third call refill the shared cache."""
    def problem(seed, B, n):
        la = rand_layout((B, n, n), 0.6, seed, ensure_rows=True)
        lmask = la & rand_layout((B, n, n), 0.7, seed + 1)
        g = torch.Generator().manual_seed(seed + 2)
        mask = torch.rand((int(lmask.sum()), sbs, sbs), generator=g) < 0.3
        full = torch.ones((B, n, 1), dtype=torch.bool)
        q, k, v = (rand_blocks(B * n, sbs, dtype, seed + s) for s in (3, 4, 5))
        go = rand_blocks(B * n, sbs, dtype, seed + 6)
        return [t.to(device) for t in (la, lmask, mask, full, q, k, v, go)]

    def forward(p, cache):
        la, lmask, mask, full, q, k, v, go = p
        leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
        out = bs.ops.flash_attention(leaves[0], full, leaves[1], full, leaves[2], full, la, sbs, attention_mask=mask,
                                     sparsity_layout_mask=lmask, layout_cache=cache)
        return out, leaves

    problems = [problem(10, 2, 4), problem(20, 2, 4), problem(30, 1, 3)]
    expected = []
    for p in problems:
        out, leaves = forward(p, {})
        expected.append(torch.autograd.grad(out, leaves, p[-1]))
    shared = {}
    runs = [forward(p, shared) for p in problems]
    for (out, leaves), p, want in zip(runs, problems, expected):
        got = torch.autograd.grad(out, leaves, p[-1])
        assert all(torch.equal(a, b) for a, b in zip(got, want))


def test_attention_refuses_a_mask_changed_in_place_before_the_backward_pass(device):
    """The mask is saved for the backward pass like an operand (blksprs/ops/flash_attention.py:498-501), so
    autograd notices a change in place."""
    sbs, lay = 64, _full(device)
    q, k, v = (rand_blocks(1, sbs, torch.bfloat16, s).to(device).requires_grad_(True) for s in (1, 2, 3))
    mask = torch.rand((1, sbs, sbs), device=device) < 0.3
    out = bs.ops.flash_attention(q, lay, k, lay, v, lay, lay, sbs, attention_mask=mask, sparsity_layout_mask=lay)
    mask.logical_not_()
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        out.float().sum().backward()


def test_attention_without_mask_facts_gives_the_same_bits(device):
    """``disable_mask_facts``: nothing is kept per mask tensor; outputs and gradients are the same bits, on the
    first call and on repeated calls with one mask and one cache."""
    sbs, B, n = 64, 2, 6
    la = rand_layout((B, n, n), 0.6, 1, ensure_rows=True)
    lmask = la & torch.ones((n, n), dtype=torch.bool).triu()
    g = torch.Generator().manual_seed(2)
    mask = torch.rand((int(lmask.sum()), sbs, sbs), generator=g) < 0.5
    mask[::2] = True  # every other mask block masks everything: pairs the facts would drop
    full = torch.ones((B, n, 2), dtype=torch.bool)
    q, k, v = (rand_blocks(B * n * 2, sbs, torch.bfloat16, s).to(device) for s in (3, 4, 5))
    go = rand_blocks(B * n * 2, sbs, torch.bfloat16, 6).to(device)
    la, lmask, mask, full = (t.to(device) for t in (la, lmask, mask, full))

    def three_steps():
        cache, results = {}, []
        for _ in range(3):
            leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
            out = bs.ops.flash_attention(leaves[0], full, leaves[1], full, leaves[2], full, la, sbs,
                                         attention_mask=mask, sparsity_layout_mask=lmask, layout_cache=cache)
            results.append((out.detach(), *torch.autograd.grad(out, leaves, go)))
        return cache, results

    cache_on, with_facts = three_steps()
    bs.utils.disable_mask_facts()
    try:
        cache_off, without = three_steps()
    finally:
        bs.utils.enable_mask_facts()
    assert "mask_facts" in cache_on and "mask_facts" not in cache_off
    for a, b in zip(with_facts, without):
        assert all(torch.equal(s, t) for s, t in zip(a, b))


def test_readme_sequence_with_compiled_matmul(device):
    """test/cases/test_readme.py: the README's tour, with ``torch.compile(bs.ops.matmul)`` in default mode."""
    b, h, m, n, k, sbs = 2, 4, 64, 64, 16, 16
    x = torch.randn((b, h, m, k), device=device)
    y = torch.randn((b, h, n, k), device=device).transpose(-1, -2).contiguous()
    x_dense, x_shape = bs.utils.do_shape_blocksparse(x)
    y_dense, _ = bs.utils.do_shape_blocksparse(y)
    lx = bs.layouting.build_sparsity_layout(x_dense, sbs)
    ly = bs.layouting.build_sparsity_layout(y_dense, sbs)
    lo = torch.ones((b * h, m // sbs, n // sbs), dtype=torch.bool, device=device)
    lo.view(-1)[torch.randperm(lo.numel(), device=device)[: lo.numel() // 4]] = False
    x_sparse, y_sparse = bs.ops.to_sparse(x_dense, lx, sbs), bs.ops.to_sparse(y_dense, ly, sbs)
    o_sparse = torch.compile(bs.ops.matmul)(x_sparse, lx, y_sparse, ly, lo, sbs)
    o_sparse = torch.add(o_sparse, 1)
    o_dense = bs.ops.to_dense(o_sparse, lo, sbs)
    o_torch = torch.add(torch.matmul(x_dense, y_dense), 1)
    round_trip = bs.ops.to_dense(bs.ops.to_sparse(o_torch, lo, sbs), lo, sbs, fill_value=0)
    assert torch.allclose(o_dense, round_trip, atol=2e-2)
    assert torch.equal(bs.layouting.build_sparsity_layout(o_dense, sbs), lo)
    assert bs.utils.undo_shape_blocksparse(o_dense, x_shape).shape == (b, h, m, n)
    bs.ops.transpose(o_sparse, lo, sbs)
    bs.ops.softmax(o_sparse, lo, sbs, flag_fused=False)
    bs.ops.softmax_fused(o_sparse, lo, sbs)
    bs.ops.softmax(o_sparse, lo, sbs)
    bs.ops.misc.row_wise_sum(o_sparse, lo, sbs)
    bs.ops.misc.row_wise_max(o_sparse, lo, sbs)

    seq, hd, sbs = 512, 64, 64
    q, kk, v = (torch.randn((b, seq, h, hd), device=device) for _ in range(3))
    qd, kd, vd = (t.transpose(1, 2).reshape(-1, seq, hd).contiguous() for t in (q, kk, v))
    lqkv = torch.ones((b * h, seq // sbs, hd // sbs), dtype=torch.bool, device=device)
    la = torch.tril(torch.ones((b * h, seq // sbs, seq // sbs), dtype=torch.bool, device=device))
    lout = bs.layouting.build_sparsity_layout_matmul(la, lqkv)
    cache = bs.ops.flash_attention_build_layout_cache(la, sparsity_layout_q=lqkv, sparsity_layout_k=lqkv,
                                                      sparsity_layout_v=lqkv, n_seq_blocks_q=seq // sbs,
                                                      n_seq_blocks_k=seq // sbs, n_head_blocks=hd // sbs,
                                                      sparsity_layout_o=lout)
    out = bs.ops.flash_attention(bs.ops.to_sparse(qd, lqkv, sbs), lqkv, bs.ops.to_sparse(kd, lqkv, sbs), lqkv,
                                 bs.ops.to_sparse(vd, lqkv, sbs), lqkv, la, sbs, layout_cache=cache,
                                 sparsity_layout_o=lout)
    dense = bs.ops.to_dense(out, lout, sbs)
    assert dense.reshape(b, h, seq, hd).transpose(1, 2).shape == (b, seq, h, hd)
    # block-causal attention on the dense tensors
    allowed = la[0].repeat_interleave(sbs, 0).repeat_interleave(sbs, 1)
    scores = (qd @ kd.transpose(-1, -2) / math.sqrt(hd)).masked_fill(~allowed, float("-inf"))
    assert_close(dense, torch.softmax(scores, -1) @ vd, 1e-4, "README attention")


@pytest.mark.parametrize("limit", [0, 4 << 30])
def test_attention_backward_of_16_bit_blocks_after_an_fp32_backward_on_the_same_cache(device, limit, monkeypatch):
    """Only the 16-bit kernels for 64 x 64 blocks write records into the backward's scratch.  An fp32 backward on the
    same cache and mask must leave nothing behind that a later bf16 backward would take for records: the bf16 call
    announces ``bwd_scratch_ready == 0`` and gives the bits of a fresh cache; the call after it may reuse its own."""
    from blksprs_amd import _capi
    from blksprs_amd.utils import validation
    monkeypatch.setattr(validation, "_kept_ds_limit", limit)
    sbs, B, n = 64, 2, 6
    la = rand_layout((B, n, n), 0.6, 1, ensure_rows=True).to(device)
    lmask = (la.cpu() & rand_layout((B, n, n), 0.7, 2)).to(device)
    mask = (torch.rand((int(lmask.sum()), sbs, sbs), generator=torch.Generator().manual_seed(3)) < 0.3).to(device)
    full = torch.ones((B, n, 1), dtype=torch.bool, device=device)
    q, k, v, go = (rand_blocks(B * n, sbs, torch.float32, s).to(device) for s in (4, 5, 6, 7))

    def grads(dtype, cache):
        leaves = [t.to(dtype).requires_grad_(True) for t in (q, k, v)]
        out = bs.ops.flash_attention(leaves[0], full, leaves[1], full, leaves[2], full, la, sbs, attention_mask=mask,
                                     sparsity_layout_mask=lmask, layout_cache=cache)
        return torch.autograd.grad(out, leaves, go.to(dtype))

    expected = grads(torch.bfloat16, {})
    seen = []
    real_call = _capi.call

    def spy(name, *args):
        if name == "bsa_attn_bwd":
            block = args[0]._obj
            seen.append((block.dtype, block.bwd_scratch_ready, block.bwd_ds_bytes))
        return real_call(name, *args)

    monkeypatch.setattr(_capi, "call", spy)
    shared = {}
    grads(torch.float32, shared)
    grads(torch.float32, shared)
    first = grads(torch.bfloat16, shared)
    second = grads(torch.bfloat16, shared)
    torch.cuda.synchronize()
    assert [s[:2] for s in seen] == [(_capi.F32, 0), (_capi.F32, 0), (_capi.BF16, 0), (_capi.BF16, 1)]
    assert all((s[2] > 0) == (limit > 0 and s[0] == _capi.BF16) for s in seen)
    for got in (first, second):
        assert all(torch.equal(a, b) for a, b in zip(got, expected))


def test_operators_under_torch_compile_run_eagerly_with_eager_results(device):
    """The public operators run eagerly: a compiled caller leaves its graph at each of them and resumes behind it,
    with the results of eager mode.  ``fullgraph=True`` either gives the same results (torch then treats the
    operator, which is marked ``torch.compiler.disable``, as an opaque call) or refuses the caller with an error
    that names the graph break; it never gives other numbers.  (The reference registers its launchers with
    ``torch.library.triton_op`` and traces through them; here the lookup tables are built and the kernels launched
    outside any trace.)"""
    import torch._dynamo
    sbs = 32
    layout = rand_layout((2, 3, 3), 0.7, 5, ensure_rows=True).to(device)
    x = rand_blocks(int(layout.sum()), sbs, torch.float32, 6).to(device)

    def caller(t):
        return bs.ops.softmax(t * 2.0, layout, sbs) + 1.0

    torch._dynamo.reset()
    eager = caller(x)
    assert torch.allclose(torch.compile(caller)(x), eager, rtol=1e-6, atol=1e-6)
    try:
        whole = torch.compile(caller, fullgraph=True)(x)
    except Exception as error:  # the error class differs between torch versions
        assert any(word in str(error).lower() for word in ("graph break", "fullgraph", "disable")), error
    else:
        assert torch.allclose(whole, eager, rtol=1e-6, atol=1e-6)
    torch._dynamo.reset()
