"""Tensors whose compressed storage crosses 2**31 - 1 elements: the cases of the reference's
test/cases/test_blocksparse.py:86-117 (configurations), :2018-2104 (conversion, transpose, matmul), :2106-2130
(layout of a dense tensor), :2620-2687 (softmax, fused and regular) and :2689-2742 (flash attention with 32768
head-dimension elements = 1024 head slices), restated against dense torch on sampled blocks, plus properties that
hold for every element and need no oracle (the dense oracle cannot hold these sizes): exact round trips, a product
with identity blocks that reproduces its operand bit for bit, softmax rows that sum to one.

Every case needs a few GiB on the card; a case is skipped, with the reason, when ``mem_get_info`` says that the
card cannot hold it."""

import pytest
import torch

import blksprs_amd as bs

pytestmark = pytest.mark.gpu

SBS = 32
# (b, m, k): compressed storage of b * (m / 32) * (k / 32) blocks of 32 x 32: just below, and exactly at, 2**31 elements
BELOW_AND_ABOVE = [(4095, 16384, 32), (4096, 16384, 32)]
ABOVE = [(4096, 16384, 32)]


def _require_free(gib):
    torch.cuda.empty_cache()  # what earlier tests left in torch's pool counts as free
    free, _ = torch.cuda.mem_get_info()
    if free < gib * (1 << 30):
        pytest.skip(f"needs {gib} GiB of free device memory, the card reports {free / (1 << 30):.1f} GiB")


def _samples(n):
    return sorted({0, 1, n // 2, n - 2, n - 1} & set(range(n)))


def _block_index(b, r, c, n_rows, n_cols):
    return (b * n_rows + r) * n_cols + c


def _dense_block(x, b, r, c=0):
    return x[b, r * SBS:(r + 1) * SBS, c * SBS:(c + 1) * SBS]


@pytest.mark.parametrize("b,m,k", BELOW_AND_ABOVE)
def test_conversion_and_transpose_across_the_limit(device, b, m, k):
    """to_sparse, to_dense and transpose with 2**31 elements of compressed storage (byte offsets beyond 2**32):
    sampled blocks against the dense tensor, the whole round trip bit for bit, and a double transpose that gives
    the compressed tensor back."""
    _require_free(24)
    assert b * m * k >= 2 ** 31 - 2 ** 19
    n_rows, n_cols = m // SBS, k // SBS
    x = torch.randn((b, m, k), device=device, dtype=torch.float16)
    layout = torch.ones((b, n_rows, n_cols), dtype=torch.bool, device=device)
    xs = bs.ops.to_sparse(x, layout, SBS)
    assert xs.shape == (b * n_rows * n_cols, SBS, SBS)
    for bi in _samples(b):
        for ri in _samples(n_rows):
            assert torch.equal(xs[_block_index(bi, ri, 0, n_rows, n_cols)], _dense_block(x, bi, ri))
    back = bs.ops.to_dense(xs, layout, SBS)
    assert torch.equal(back, x)
    del back
    xt, layout_t = bs.ops.transpose(xs, layout, SBS)
    assert layout_t.shape == (b, n_cols, n_rows)
    for bi in _samples(b):
        for ri in _samples(n_rows):
            assert torch.equal(xt[_block_index(bi, 0, ri, n_cols, n_rows)], _dense_block(x, bi, ri).T)
    del x
    xtt, layout_tt = bs.ops.transpose(xt, layout_t, SBS)
    assert torch.equal(layout_tt, layout) and torch.equal(xtt, xs)


@pytest.mark.parametrize("b,m,k", BELOW_AND_ABOVE)
def test_layout_of_a_dense_tensor_across_the_limit(device, b, m, k):
    """build_sparsity_layout of a dense tensor of 2**31 elements: blocks zeroed at the far end of the tensor are
    found, all others are active."""
    _require_free(8)
    n_rows = m // SBS
    x = torch.ones((b, m, k), device=device, dtype=torch.float16)
    expected = torch.ones((b, n_rows, k // SBS), dtype=torch.bool, device=device)
    for bi in _samples(b):
        for ri in _samples(n_rows)[1::2]:
            _dense_block(x, bi, ri).zero_()
            expected[bi, ri, 0] = False
    assert torch.equal(bs.layouting.build_sparsity_layout(x, SBS), expected)


@pytest.mark.parametrize("b,m,k", ABOVE)
def test_matmul_across_the_limit(device, b, m, k):
    """x (2**31 elements, one block column) times y (one 32 x 32 block per batch entry): sampled output blocks
    against dense torch at 2e-2, and, with identity blocks for y, an output that equals x bit for bit everywhere."""
    _require_free(24)
    n_rows = m // SBS
    x = torch.randn((b * n_rows, SBS, SBS), device=device, dtype=torch.float16)
    y = torch.randn((b, SBS, SBS), device=device, dtype=torch.float16)
    lx = torch.ones((b, n_rows, 1), dtype=torch.bool, device=device)
    ly = torch.ones((b, 1, 1), dtype=torch.bool, device=device)
    cache = {}
    out = bs.ops.matmul(x, lx, y, ly, lx, SBS, layout_cache=cache)
    assert out.shape == x.shape
    for bi in _samples(b):
        for ri in _samples(n_rows):
            at = _block_index(bi, ri, 0, n_rows, 1)
            want = (x[at].float() @ y[bi].float()).half()
            assert torch.allclose(out[at].float(), want.float(), rtol=2e-2, atol=2e-2), (bi, ri)
    del out
    eye = torch.eye(SBS, device=device, dtype=torch.float16).expand(b, SBS, SBS).contiguous()
    same = bs.ops.matmul(x, lx, eye, ly, lx, SBS, layout_cache=cache)
    assert torch.equal(same, x)


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("b,m,k", ABOVE)
def test_softmax_across_the_limit(device, fused, b, m, k):
    """fp32 softmax over 2**31 elements (8 GiB in, 8 GiB out), fused and regular: sampled blocks against
    torch.softmax at 1e-5, and for every row of the tensor: entries in [0, 1] that sum to one."""
    _require_free(28)
    n_rows = m // SBS
    x = torch.randn((b * n_rows, SBS, SBS), device=device, dtype=torch.float32)
    layout = torch.ones((b, n_rows, 1), dtype=torch.bool, device=device)
    out = bs.ops.softmax(x, layout, SBS, flag_fused=fused)
    for bi in _samples(b):
        for ri in _samples(n_rows):
            at = _block_index(bi, ri, 0, n_rows, 1)
            assert torch.allclose(out[at], torch.softmax(x[at], dim=-1), rtol=1e-5, atol=1e-5), (bi, ri)
    del x
    sums = out.sum(dim=-1)
    assert float((sums - 1).abs().max()) < 1e-4
    assert float(out.min()) >= 0.0 and float(out.max()) <= 1.0


def test_flash_attention_with_1024_head_slices_across_the_limit(device):
    """b = 2048 sequences of one 32-token block with head dimension 32768 (q and k hold 2**31 elements each in
    1024 head slices): the output of sampled batch entries against softmax(q k^T / sqrt(d)) v in fp32."""
    _require_free(24)
    b, m, n, k = 2048, 32, 32, 32768
    q = torch.randn((b, m, k), device=device, dtype=torch.float16)
    key = torch.randn((b, m, k), device=device, dtype=torch.float16)
    v = torch.randn((b, m, n), device=device, dtype=torch.float16)
    lq = torch.ones((b, m // SBS, k // SBS), dtype=torch.bool, device=device)
    lv = torch.ones((b, m // SBS, n // SBS), dtype=torch.bool, device=device)
    la = torch.ones((b, m // SBS, m // SBS), dtype=torch.bool, device=device)
    picks = _samples(b)
    refs = []
    for bi in picks:
        scores = (q[bi].float() @ key[bi].float().T) / k ** 0.5
        refs.append(torch.softmax(scores, dim=-1) @ v[bi].float())
    qs = bs.ops.to_sparse(q, lq, SBS)
    del q
    ks = bs.ops.to_sparse(key, lq, SBS)
    del key
    vs = bs.ops.to_sparse(v, lv, SBS)
    out = bs.ops.flash_attention(qs, lq, ks, lq, vs, lv, la, SBS, sparsity_layout_o=lv)
    dense = bs.ops.to_dense(out, lv, SBS)
    for bi, want in zip(picks, refs):
        assert torch.allclose(dense[bi].float(), want, rtol=2e-2, atol=2e-2), bi


def test_bf16_matmul_and_its_gradients_across_the_limit_with_64_blocks(device):
    """The kernels for 16-bit operands and 64 x 64 blocks (rows of the output in the forward pass, lines of the
    output gradient in the backward pass) on 563 200 blocks = 2.3 * 10**9 elements per tensor: with identity blocks
    for y the product and dX reproduce x and dO bit for bit everywhere; dY of sampled batch entries against dense
    torch (512 blocks of dO per column: the longest line the line kernel takes)."""
    _require_free(40)
    sbs, b, n_rows = 64, 1100, 512
    g = torch.Generator(device=device).manual_seed(0)
    x = torch.randn((b * n_rows, sbs, sbs), device=device, dtype=torch.bfloat16, generator=g)
    assert x.numel() > 2 ** 31
    eye = torch.eye(sbs, device=device, dtype=torch.bfloat16).expand(b, sbs, sbs).contiguous()
    lx = torch.ones((b, n_rows, 1), dtype=torch.bool, device=device)
    ly = torch.ones((b, 1, 1), dtype=torch.bool, device=device)
    xg, yg = x.requires_grad_(True), eye.requires_grad_(True)
    cache = {}
    out = bs.ops.matmul(xg, lx, yg, ly, lx, sbs, layout_cache=cache)
    assert torch.equal(out.detach(), x.detach())
    go = torch.randn(out.shape, device=device, dtype=torch.bfloat16, generator=g) / 32
    dx, dy = torch.autograd.grad(out, (xg, yg), go)
    assert "grad_x_part_table" in cache and int(cache["grad_lines_error"][0].item()) == 0
    assert torch.equal(dx, go)
    for bi in _samples(b):
        rows = slice(bi * n_rows, (bi + 1) * n_rows)
        want = torch.einsum("nrk,nrc->kc", x.detach()[rows].float(), go[rows].float())
        assert torch.allclose(dy[bi].float(), want, rtol=2e-2, atol=2e-2), bi
