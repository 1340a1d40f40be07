"""Parity of block-sparse flash attention (forward and backward) with the CPU oracle:
rtol = atol = 1e-5 for fp32... the oracle is dense fp64 here, so fp32 is checked at 2e-5 absolute on
O(1) values; 2e-2 for fp16 / bf16."""

import math

import pytest
import torch
import torch.nn.functional as F

import blksprs_amd as bs
from oracle import blksprs_oracle as orc
from tests.helpers import assert_close, rand_blocks, rand_layout

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def _run_case(device, dtype, sbs, B, nq, nk, nh, nhv, density, seed, use_mask=False, use_bias=False,
              use_causal=False, sparse_heads=False, custom_o=False, scale=None):
    g = torch.Generator().manual_seed(seed)
    la = orc.random_layout((B, nq, nk), density, g, ensure_rows=True)
    full = lambda r, c: torch.ones((B, r, c), dtype=torch.bool)
    lq, lk, lv = full(nq, nh), full(nk, nh), full(nk, nhv)
    if sparse_heads:
        lq = orc.random_layout((B, nq, nh), 0.7, g, ensure_rows=True)
        lk = orc.random_layout((B, nk, nh), 0.7, g, ensure_rows=True)
        lv = orc.random_layout((B, nk, nhv), 0.7, g, ensure_rows=True)
    lo = orc.random_layout((B, nq, nhv), 0.8, g, ensure_rows=True) if custom_o else None
    q = rand_blocks(int(lq.sum()), sbs, dtype, seed + 1)
    k = rand_blocks(int(lk.sum()), sbs, dtype, seed + 2)
    v = rand_blocks(int(lv.sum()), sbs, dtype, seed + 3)
    mask = lmask = bias = lbias = lengths = None
    if use_mask:
        lmask = la & orc.random_layout((B, nq, nk), 0.7, g)
        mask = torch.rand((int(lmask.sum()), sbs, sbs), generator=g) < 0.3
    if use_bias:
        lbias = la & orc.random_layout((B, nq, nk), 0.7, g)
        bias = rand_blocks(int(lbias.sum()), sbs, dtype, seed + 4)
    if use_causal:
        lengths = torch.randint(1, nq * sbs + 1, (B,), generator=g)
        lengths[0] = nq * sbs

    to = lambda t: None if t is None else t.to(device)
    qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
    bd = None if bias is None else bias.to(device).requires_grad_(True)
    out = bs.ops.flash_attention(qd, to(lq), kd, to(lk), vd, to(lv), to(la), sbs, scale=scale,
                                 attention_mask=to(mask), sparsity_layout_mask=to(lmask),
                                 attention_bias=bd, sparsity_layout_bias=to(lbias),
                                 sparsity_layout_o=to(lo), causal_lengths=to(lengths))
    assert isinstance(out, bs.BlksprsTensor) and out.dtype == dtype

    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    b64 = None if bias is None else bias.double().requires_grad_(True)
    ref = orc.flash_attention(q64, lq.numpy(), k64, lk.numpy(), v64, lv.numpy(), la.numpy(), sbs, scale=scale,
                              mask=mask, layout_mask=None if lmask is None else lmask.numpy(),
                              bias=b64, layout_bias=None if lbias is None else lbias.numpy(),
                              layout_o=None if lo is None else lo.numpy(), causal_lengths=lengths,
                              acc_dtype=torch.float64)
    tol = TOL[dtype]
    tag = f"{dtype} sbs={sbs} mask={use_mask} bias={use_bias} causal={use_causal}"
    assert_close(out, ref, tol, "O " + tag)
    go = rand_blocks(out.size(0), sbs, dtype, seed + 5)
    out.backward(go.to(device))
    ref.backward(go.double())
    gtol = tol
    assert_close(qd.grad, q64.grad, gtol, "dQ " + tag)
    assert_close(kd.grad, k64.grad, gtol, "dK " + tag)
    assert_close(vd.grad, v64.grad, gtol, "dV " + tag)
    if bias is not None:
        assert_close(bd.grad, b64.grad, gtol, "dBias " + tag)
    return qd.grad, kd.grad, vd.grad


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sbs", [16, 32, 64])
def test_plain_layout(device, dtype, sbs):
    _run_case(device, dtype, sbs, B=2, nq=4, nk=4, nh=2, nhv=2, density=0.5, seed=sbs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sbs", [16, 64])
@pytest.mark.parametrize("use_mask,use_bias,use_causal", [(True, False, False), (False, True, False),
                                                           (False, False, True), (True, True, True)])
def test_mask_bias_causal(device, dtype, sbs, use_mask, use_bias, use_causal):
    _run_case(device, dtype, sbs, B=2, nq=3, nk=3, nh=1, nhv=2, density=0.7, seed=3 * sbs + use_mask,
              use_mask=use_mask, use_bias=use_bias, use_causal=use_causal)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_rectangular_sparse_heads_and_custom_output_layout(device, dtype):
    _run_case(device, dtype, 32, B=2, nq=3, nk=5, nh=3, nhv=2, density=0.5, seed=77, sparse_heads=True,
              custom_o=True, use_mask=True, use_bias=True, scale=0.37)


@pytest.mark.parametrize("dtype,sbs", [(torch.float32, 16), (torch.float32, 64), (torch.bfloat16, 32), (torch.float16, 16)])
@pytest.mark.parametrize("nh,nhv", [(4, 3), (1, 4), (3, 5)])
def test_many_head_slices_and_long_key_lists(device, dtype, sbs, nh, nhv):
    """The fp32 matrix-core forward kernel: key lists longer than its groups of waves (9 key blocks for 2 or 4
    groups, rows with a single key block next to them), three and four value head slices (the kernel is built for
    1, 2 and 4), and five, which it leaves to the generic kernel; sparse head layouts, mask, bias and causal
    lengths together."""
    _run_case(device, dtype, sbs, B=2, nq=5, nk=9, nh=nh, nhv=nhv, density=0.55, seed=sbs + nh, use_mask=True,
              use_bias=True, sparse_heads=True, custom_o=True)
    _run_case(device, dtype, sbs, B=1, nq=9, nk=9, nh=nh, nhv=nhv, density=0.3, seed=sbs + nhv, use_causal=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("use_mask,use_bias,use_causal,nh,nhv", [(False, False, False, 2, 2), (True, True, False, 1, 2),
                                                               (False, False, True, 2, 1)])
def test_dk_dv_of_more_key_blocks_than_workgroups(device, dtype, use_mask, use_bias, use_causal, nh, nhv):
    """The dK / dV kernel keeps one workgroup per compute unit for the whole launch; a workgroup walks key block
    after key block (drawn by ticket), with the next block's K / V and first tile requested during the current
    one.  400 (or 270) key rows are 50 (34) per XCD against 32 workgroups; at 8 % density most key blocks are attended by no
    query block or by one (blocks without tiles and with a single tile take paths of their own), a few by
    several."""
    B, nq, nk = (3, 90, 90) if use_causal else (4, 12, 100)  # the native causal predicate wants a square layout
    _run_case(device, dtype, 64, B, nq, nk, nh, nhv, 0.08, seed=23, use_mask=use_mask, use_bias=use_bias,
              use_causal=use_causal)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("use_mask,use_bias,use_causal,nh,nhv", [(False, False, False, 2, 2), (True, True, False, 1, 2),
                                                               (False, False, True, 2, 1), (True, False, True, 1, 1)])
def test_backward_without_room_for_ds_forms_it_twice(device, dtype, use_mask, use_bias, use_causal, nh, nhv, monkeypatch):
    """With room in the scratch the dK / dV kernel leaves dS of every pair behind and dQ = dS K is a product of its
    own (the path every other backward test of 64 x 64 16-bit blocks takes); without, the dQ kernel forms the scores
    and dS a second time.  Both against the oracle, and the two against each other."""
    from blksprs_amd.utils import validation
    B, nq, nk = (2, 24, 24) if use_causal else (2, 12, 40)
    kwargs = dict(seed=31, use_mask=use_mask, use_bias=use_bias, use_causal=use_causal)
    kept = _run_case(device, dtype, 64, B, nq, nk, nh, nhv, 0.3, **kwargs)
    monkeypatch.setattr(validation, "_kept_ds_limit", 0)
    twice = _run_case(device, dtype, 64, B, nq, nk, nh, nhv, 0.3, **kwargs)
    for name, a, b in zip(("dQ", "dK", "dV"), kept, twice):
        assert_close(a, b.double(), 1e-2, f"{name}, dS kept against dS formed twice")


def test_bigbird_layout_with_causal_mask_head_dim_128(device):
    """Config 4's shape at reduced batch and length: bf16, sbs 64, head_dim 128, BigBird layout, causal mask."""
    B, n, sbs, nh = 2, 16, 64, 2
    g = torch.Generator().manual_seed(0)
    la = orc.bigbird_layout(B, n, g)
    lmask = la & torch.ones((n, n), dtype=torch.bool).triu()
    pos = torch.arange(n * sbs)
    dense_mask = (pos.view(1, -1) > pos.view(-1, 1)).unsqueeze(0).expand(B, -1, -1)
    mask = orc.to_sparse(dense_mask, lmask.numpy(), sbs)
    full = torch.ones((B, n, nh), dtype=torch.bool)
    q, k, v = (rand_blocks(B * n * nh, sbs, torch.bfloat16, s) for s in (1, 2, 3))
    qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
    out = bs.ops.flash_attention(qd, full.to(device), kd, full.to(device), vd, full.to(device), la.to(device), sbs,
                                 attention_mask=mask.to(device), sparsity_layout_mask=lmask.to(device))
    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    ref = orc.flash_attention(q64, full.numpy(), k64, full.numpy(), v64, full.numpy(), la.numpy(), sbs,
                              mask=mask, layout_mask=lmask.numpy(), acc_dtype=torch.float64)
    assert_close(out, ref, 2e-2, "O bigbird")
    # same result from the native causal predicate instead of the mask tensor
    out2 = bs.ops.flash_attention(qd, full.to(device), kd, full.to(device), vd, full.to(device), la.to(device), sbs,
                                  causal_lengths=torch.full((B,), n * sbs, device=device))
    assert_close(out2, ref, 2e-2, "O bigbird, causal_lengths")
    go = rand_blocks(out.size(0), sbs, torch.bfloat16, 5)
    out.backward(go.to(device))
    ref.backward(go.double())
    assert_close(qd.grad, q64.grad, 2e-2, "dQ bigbird")
    assert_close(kd.grad, k64.grad, 2e-2, "dK bigbird")
    assert_close(vd.grad, v64.grad, 2e-2, "dV bigbird")


def test_full_layout_equals_sdpa(device):
    # reference: test_regressions.py:488-527
    B, S, D, sbs = 2, 128, 64, 32
    q, k, v = (torch.randn((B, S, D), device=device) for _ in range(3))
    lay = torch.ones((B, S // sbs, D // sbs), dtype=torch.bool, device=device)
    la = torch.ones((B, S // sbs, S // sbs), dtype=torch.bool, device=device)
    out = bs.ops.flash_attention(bs.ops.to_sparse(q, lay, sbs), lay, bs.ops.to_sparse(k, lay, sbs), lay,
                                 bs.ops.to_sparse(v, lay, sbs), lay, la, sbs)
    expected = F.scaled_dot_product_attention(q.double().cpu(), k.double().cpu(), v.double().cpu())
    assert_close(bs.ops.to_dense(out, lay, sbs), expected, 1e-5, "sdpa")


@pytest.mark.parametrize("dtype,n_key_blocks", [(torch.bfloat16, 256), (torch.float16, 1024)])
def test_uniform_attention_over_a_long_sequence_is_exact(device, dtype, n_key_blocks):
    # reference: test_regressions.py:63-94 - q = k = 0, v = 1 must give exactly 1
    sbs = 64
    lq = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    lk = torch.ones((1, n_key_blocks, 1), dtype=torch.bool, device=device)
    la = torch.ones((1, 1, n_key_blocks), dtype=torch.bool, device=device)
    q = torch.zeros((1, sbs, sbs), device=device, dtype=dtype)
    k = torch.zeros((n_key_blocks, sbs, sbs), device=device, dtype=dtype)
    v = torch.ones((n_key_blocks, sbs, sbs), device=device, dtype=dtype)
    out = bs.ops.flash_attention(q, lq, k, lk, v, lk, la, sbs)
    assert torch.all(out == 1)


def test_uniform_gradient_over_many_queries_is_exact(device):
    # reference: test_regressions.py:97-129 - dV = n_queries / n_keys exactly
    sbs, nq = 64, 256
    lq = torch.ones((1, nq, 1), dtype=torch.bool, device=device)
    lk = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    la = torch.ones((1, nq, 1), dtype=torch.bool, device=device)
    q = torch.zeros((nq, sbs, sbs), device=device, dtype=torch.bfloat16)
    k = torch.zeros((1, sbs, sbs), device=device, dtype=torch.bfloat16)
    v = torch.ones((1, sbs, sbs), device=device, dtype=torch.bfloat16, requires_grad=True)
    bs.ops.flash_attention(q, lq, k, lk, v, lk, la, sbs).sum().backward()
    assert torch.all(v.grad == nq)


def test_mask_beats_infinite_bias_and_fully_masked_rows_are_zero(device):
    # reference: test_regressions.py:2075-2120
    sbs = 16
    lay = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    q, k, v = (torch.randn((1, sbs, sbs), device=device, requires_grad=True) for _ in range(3))
    bias = torch.zeros((1, sbs, sbs), device=device)
    bias[0, :, 0] = float("inf")
    bias.requires_grad_(True)
    mask = torch.zeros((1, sbs, sbs), dtype=torch.bool, device=device)
    mask[0, :, 0] = True
    mask[0, 5, :] = True
    out = bs.ops.flash_attention(q, lay, k, lay, v, lay, lay, sbs, attention_mask=mask, sparsity_layout_mask=lay,
                                 attention_bias=bias, sparsity_layout_bias=lay)
    assert torch.isfinite(out).all() and torch.all(out[0, 5] == 0)
    out.sum().backward()
    for t in (q, k, v, bias):
        assert torch.isfinite(t.grad).all()
    assert torch.all(bias.grad[0, :, 0] == 0) and torch.all(bias.grad[0, 5] == 0)


def test_zero_width_qk_head_dimension(device):
    # reference: test_regressions.py:1256-1283 - no q/k blocks: scores are zero, scale defaults to 1
    sbs = 16
    lq = torch.ones((1, 2, 0), dtype=torch.bool, device=device)
    lv = torch.ones((1, 2, 1), dtype=torch.bool, device=device)
    la = torch.ones((1, 2, 2), dtype=torch.bool, device=device)
    e = torch.empty((0, sbs, sbs), device=device)
    v = torch.randn((2, sbs, sbs), device=device)
    out = bs.ops.flash_attention(e, lq, e, lq, v, lv, la, sbs)
    mean = v.reshape(2 * sbs, sbs).mean(dim=0)
    assert torch.isfinite(out).all()
    assert_close(out, mean.expand(2, sbs, sbs), 1e-5, "zero head dim")
    same = bs.ops.flash_attention(e, lq, e, lq, v, lv, la, sbs, scale=1.0)
    assert torch.equal(out, same)


def test_default_output_layout_and_cache_reuse(device):
    # reference: test_regressions.py:450-532
    sbs, B = 16, 1
    la = torch.tensor([[[1, 0], [0, 0]]], dtype=torch.bool, device=device)
    lay = torch.ones((B, 2, 1), dtype=torch.bool, device=device)
    q, k, v = (torch.randn((2, sbs, sbs), device=device) for _ in range(3))
    cache = bs.ops.flash_attention_build_layout_cache(la, lay, lay, lay)
    assert torch.equal(cache["sparsity_layout_o"].cpu(), torch.tensor([[[True], [False]]]))
    assert cache["key_indices"].dtype == torch.int32 and cache["query_offsets"].dtype == torch.int32
    assert cache["max_keys_per_query"] == 1 and cache["n_sparse_blocks_o"] == 1 and cache["n_sparse_blocks_q"] == 2
    kept = cache["key_indices"]
    out = bs.ops.flash_attention(q, lay, k, lay, v, lay, la, sbs, layout_cache=cache)
    assert cache["key_indices"] is kept and out.shape == (1, sbs, sbs)
    # positional order of the builder's arguments (reference: test_regressions.py:477-485)
    again = bs.ops.flash_attention_build_layout_cache(la, lay, lay, lay, 2, 2, 1, None, 1, cache)
    assert again is cache


def test_validation_errors(device):
    sbs = 16
    lay = torch.ones((1, 1, 1), dtype=torch.bool, device=device)
    t = torch.randn((1, sbs, sbs), device=device)
    with pytest.raises(ValueError, match="provided together"):
        bs.ops.flash_attention(t, lay, t, lay, t, lay, lay, sbs, attention_mask=t)
    with pytest.raises(ValueError, match="provided together"):
        bs.ops.flash_attention(t, lay, t, lay, t, lay, lay, sbs, sparsity_layout_bias=lay)
    with pytest.raises(TypeError, match="real number or None"):
        bs.ops.flash_attention(t, lay, t, lay, t, lay, lay, sbs, scale="1")
    with pytest.raises(ValueError, match="0 or 1"):
        bs.ops.flash_attention(t, lay, t, lay, t, lay, lay, sbs, attention_mask=t * 3, sparsity_layout_mask=lay)
    big = torch.randn((1, 128, 128), device=device)
    with pytest.raises(ValueError, match="at most 64"):
        bs.ops.flash_attention(big, lay, big, lay, big, lay, lay, 128)
    with pytest.raises(ValueError, match="K sparsity layout must be compatible"):
        bs.ops.flash_attention(t, lay, torch.randn((2, sbs, sbs), device=device),
                               torch.ones((1, 1, 2), dtype=torch.bool, device=device), t, lay, lay, sbs)
    with pytest.raises(TypeError, match="integral dtype"):
        bs.ops.flash_attention(t, lay, t, lay, t, lay, lay, sbs, causal_lengths=torch.ones(1, device=device))
    with pytest.raises(ValueError, match="between zero and 16"):
        bs.ops.flash_attention(t, lay, t, lay, t, lay, lay, sbs,
                               causal_lengths=torch.tensor([17], device=device))
    import numpy as np
    out = bs.ops.flash_attention(t, lay, t, lay, t, lay, lay, sbs, scale=np.float32(0.5))
    assert out.shape == (1, sbs, sbs)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nq,nh,nhv", [(7, 2, 2), (6, 1, 2), (5, 2, 1), (8, 1, 1)])
def test_matrix_core_forward_odd_sequences_and_head_slice_counts(device, dtype, nq, nh, nhv):
    _run_case(device, dtype, 64, 2, nq, 6, nh, nhv, 0.5, 70 + nq, use_mask=True, use_causal=(nq == 6))


def test_pair_lists_cover_the_layout_and_masked_tiles_change_nothing(device):
    """The forward kernel walks, per pair of query blocks, the union of their key lists.  Every active block of
    the layout appears once with its flag; whole mask blocks that are set are fetched but not computed."""
    g = torch.Generator().manual_seed(5)
    B, nq, nk, nh, sbs = 3, 9, 11, 2, 64
    la = orc.random_layout((B, nq, nk), 0.6, g, ensure_rows=True)
    full = torch.ones((B, nq, nh), dtype=torch.bool)
    fullk = torch.ones((B, nk, nh), dtype=torch.bool)
    q = rand_blocks(B * nq * nh, sbs, torch.bfloat16, 1)
    k = rand_blocks(B * nk * nh, sbs, torch.bfloat16, 2)
    v = rand_blocks(B * nk * nh, sbs, torch.bfloat16, 3)
    lmask = la.clone()
    mask = torch.rand((int(lmask.sum()), sbs, sbs), generator=g) < 0.5
    mask[::3] = True
    cache = {}
    out = bs.ops.flash_attention(q.to(device), full.to(device), k.to(device), fullk.to(device), v.to(device),
                                 fullk.to(device), la.to(device), sbs, attention_mask=mask.to(device),
                                 sparsity_layout_mask=lmask.to(device), layout_cache=cache)
    assert cache["group_size"] == 2
    records = cache["group_records"].view(-1, 16).cpu()
    entries = records[:, 0]
    assert int(((entries >> 28) & 1).sum() + ((entries >> 29) & 1).sum()) == int(la.sum())
    # records against a host restatement: packed indices of K, V and of the mask block of either query block
    offsets = cache["group_offsets"].cpu()
    pidx_mask = (torch.cumsum(lmask.reshape(-1).long(), 0) - 1).masked_fill(~lmask.reshape(-1), -1).view(B, nq, nk)
    for grp in range(B * ((nq + 1) // 2)):
        b_, p_ = divmod(grp, (nq + 1) // 2)
        keys = sorted(set(torch.nonzero(la[b_, 2 * p_]).flatten().tolist())
                      | (set(torch.nonzero(la[b_, 2 * p_ + 1]).flatten().tolist()) if 2 * p_ + 1 < nq else set()))
        got = records[offsets[grp]:offsets[grp + 1]]
        assert (got[:, 0] & 0x0fffffff).tolist() == keys
        for rec in got.tolist():
            kb = rec[0] & 0x0fffffff
            assert rec[1:5] == [(b_ * nk + kb) * nh, (b_ * nk + kb) * nh + 1] * 2
            for half in range(2):
                qb = 2 * p_ + half
                active = qb < nq and bool(la[b_, qb, kb])
                assert bool((rec[0] >> (28 + half)) & 1) == active
                assert rec[5 + half] == (int(pidx_mask[b_, qb, kb]) if active else -1)
                assert rec[7 + half] == -1
    ref = orc.flash_attention(q.double(), full.numpy(), k.double(), fullk.numpy(), v.double(), fullk.numpy(),
                              la.numpy(), sbs, mask=mask, layout_mask=lmask.numpy(), acc_dtype=torch.float64)
    assert_close(out, ref, 2e-2, "O pair lists")


def test_config4_full_size_against_sampled_oracle_rows_and_invariants(device):
    """Configuration 4 at full size (bf16, 64 heads, 8192 positions, head_dim 128, sbs 64, BigBird layout with
    causal mask blocks), where the oracle cannot run whole.  A query block row depends only on its own row of
    the layout, so the oracle is run on single rows (1 x 1 x 128 layouts against all keys of the head) and gives
    the exact output and dQ of those rows; a key block's dK and dV depend only on the rows that attend to it, so
    the oracle on the sub-layout of those rows gives them exactly.  Everything else is held to invariants of attention:
    rows of P sum to 1, hence with V = 1 the output is 1 and sum_k dV[k, f] = sum_q dO[q, f];
    rows of dS sum to 0, hence sum_k dK[k, f] = 0; and two runs give identical bits (no atomics)."""
    BH, n, sbs, nh = 64, 128, 64, 2
    g = torch.Generator().manual_seed(0)
    la = orc.bigbird_layout(BH, n, g)
    lmask = la & torch.ones((n, n), dtype=torch.bool).triu()
    lad, lmd = la.to(device), lmask.to(device)
    full = torch.ones((BH, n, nh), dtype=torch.bool, device=device)
    midx = torch.nonzero(lmd)
    r = torch.arange(sbs, device=device)
    mask = (midx[:, 2].view(-1, 1, 1) * sbs + r.view(1, 1, -1)) > (midx[:, 1].view(-1, 1, 1) * sbs + r.view(1, -1, 1))
    gd = torch.Generator(device=device).manual_seed(1)
    q, k, v, go = (torch.randn((BH * n * nh, sbs, sbs), device=device, generator=gd).to(torch.bfloat16)
                   for _ in range(4))
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    cache = {}

    def run(values):
        return bs.ops.flash_attention(q, full, k, full, values, full, lad, sbs, attention_mask=mask,
                                      sparsity_layout_mask=lmd, layout_cache=cache)

    out = run(v)
    out.backward(go)
    dq, dk, dv = q.grad.clone(), k.grad.clone(), v.grad.clone()
    q.grad = k.grad = v.grad = None
    out2 = run(v)
    out2.backward(go)
    assert torch.equal(out, out2) and torch.equal(dq, q.grad) and torch.equal(dk, k.grad) and torch.equal(dv, v.grad)

    # sampled rows against the oracle (output and dQ)
    mask_offsets = torch.cumsum(lmask.flatten().long(), 0) - 1
    for h, i in ((0, 0), (0, 127), (17, 64), (63, 1), (40, 101)):
        rows = slice((h * n + i) * nh, (h * n + i + 1) * nh)
        head = slice(h * n * nh, (h + 1) * n * nh)
        cols = torch.nonzero(lmask[h, i]).flatten()
        mk = mask[mask_offsets[(h * n + i) * n + cols]].cpu() if len(cols) else None
        q64 = q[rows].detach().cpu().double().requires_grad_(True)
        ones = lambda a, b: torch.ones((1, a, b), dtype=torch.bool).numpy()
        ref = orc.flash_attention(q64, ones(1, nh), k[head].detach().cpu().double(), ones(n, nh),
                                  v[head].detach().cpu().double(), ones(n, nh), la[h:h + 1, i:i + 1].numpy(), sbs,
                                  mask=mk, layout_mask=lmask[h:h + 1, i:i + 1].numpy() if mk is not None else None,
                                  acc_dtype=torch.float64)
        assert_close(out[rows], ref, 2e-2, f"O head {h} row {i}")
        ref.backward(go[rows].cpu().double())
        assert_close(dq[rows], q64.grad, 2e-2, f"dQ head {h} row {i}")

    # sampled key blocks against the oracle (dK and dV): a key block's gradients come from the query block rows that
    # attend to it, and those rows need all of their keys (for their softmax): the oracle runs on the sub-layout
    # of exactly those rows, whose dK / dV of that key block are then complete.  Key block 1 is a global one (every
    # later query block attends to it), the others have a handful of rows.
    for h, j in ((0, 5), (21, 1), (63, 127), (40, 64)):
        rows_of = torch.nonzero(la[h, :, j]).flatten()
        head = slice(h * n * nh, (h + 1) * n * nh)
        pick = torch.cat([torch.arange((h * n + int(i)) * nh, (h * n + int(i) + 1) * nh) for i in rows_of])
        sub_layout = la[h, rows_of][None]
        sub_lmask = lmask[h, rows_of][None]
        mask_at = torch.cat([mask_offsets[(h * n + int(i)) * n + torch.nonzero(lmask[h, int(i)]).flatten()] for i in rows_of])
        mk = mask[mask_at.to(device)].cpu() if len(mask_at) else None
        ones = lambda a, b: torch.ones((1, a, b), dtype=torch.bool).numpy()
        k64 = k[head].detach().cpu().double().requires_grad_(True)
        v64 = v[head].detach().cpu().double().requires_grad_(True)
        ref = orc.flash_attention(q[pick.to(device)].detach().cpu().double(), ones(len(rows_of), nh), k64, ones(n, nh),
                                  v64, ones(n, nh), sub_layout.numpy(), sbs, mask=mk,
                                  layout_mask=sub_lmask.numpy() if mk is not None else None, acc_dtype=torch.float64)
        ref.backward(go[pick.to(device)].cpu().double())
        mine = slice((h * n + j) * nh, (h * n + j + 1) * nh)
        assert_close(dk[mine], k64.grad[j * nh:(j + 1) * nh], 2e-2, f"dK head {h} key block {j}")
        assert_close(dv[mine], v64.grad[j * nh:(j + 1) * nh], 2e-2, f"dV head {h} key block {j}")

    # invariants over all heads
    with torch.no_grad():
        unit = run(torch.ones_like(v))
        assert float((unit.float() - 1).abs().max()) <= 2e-2
        per_head = lambda t: t.detach().float().reshape(BH, n, nh, sbs, sbs).permute(0, 1, 3, 2, 4).reshape(BH, n * sbs, nh * sbs)
        dv_h, go_h, dk_h = per_head(dv), per_head(go), per_head(dk)
        mass, want = dv_h.sum(1), go_h.sum(1)
        assert float((mass - want).abs().max()) <= 2e-2 * float(go_h.abs().sum(1).max())
        assert float(dk_h.sum(1).abs().max()) <= 2e-2 * float(dk_h.abs().sum(1).max())


def test_mask_blocks_that_mask_everything_are_found(device):
    import ctypes

    from blksprs_amd import _capi
    g = torch.Generator().manual_seed(3)
    mask = (torch.rand((37, 64, 64), generator=g) < 0.5).to(device)
    mask[::5] = True
    mask[7, 63, 63] = False  # one open position keeps a block alive
    mask[12] = True
    dead = torch.full((37,), 7, dtype=torch.uint8, device=device)
    _capi.call("bsa_attn_mask_dead", _capi.ptr(mask.view(torch.uint8)), 37, 64, _capi.ptr(dead), _capi.stream(device))
    assert torch.equal(dead.bool(), mask.view(37, -1).all(dim=1))
    assert not bool(dead[7]) and bool(dead[12]) and bool(dead[35])


@pytest.mark.parametrize("use_causal", [False, True])
def test_lists_kept_per_mask_follow_the_mask(device, use_causal):
    """From the second call with one mask tensor on, the forward walks lists without the pairs whose mask block
    masks everything and the backward reads the records of the call before.  Every call gives the bits of the
    first one; a mask changed in place, another mask tensor and other causal lengths give what a fresh cache
    gives."""
    g = torch.Generator().manual_seed(21)
    B, n, nh, sbs = 2, 8, 2, 64
    la = orc.random_layout((B, n, n), 0.7, g, ensure_rows=True).to(device)
    full = torch.ones((B, n, nh), dtype=torch.bool, device=device)
    q, k, v = (rand_blocks(B * n * nh, sbs, torch.bfloat16, s).to(device) for s in (1, 2, 3))
    lmask = la.clone()
    lmask[0, 3] = False
    n_mask = int(lmask.sum())

    def new_mask(seed):
        gm = torch.Generator().manual_seed(seed)
        m = torch.rand((n_mask, sbs, sbs), generator=gm) < 0.4
        m[torch.rand(n_mask, generator=gm) < 0.4] = True  # dead pairs
        rows = torch.cumsum(lmask.reshape(-1).long().cpu(), 0).view(B, n, n)
        m[rows[1, 1, -1]:rows[1, 2, -1]] = True  # a query block with nothing left (its blocks are contiguous)
        return m.to(device)

    def run(mask, lengths, cache):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = bs.ops.flash_attention(qq, full, kk, full, vv, full, la, sbs, attention_mask=mask,
                                     sparsity_layout_mask=lmask, layout_cache=cache, causal_lengths=lengths)
        out.backward(go)
        return out.detach(), qq.grad, kk.grad, vv.grad

    go = rand_blocks(B * n * nh, sbs, torch.bfloat16, 4).to(device)

    def same(a, b):
        for x, y in zip(a, b):
            assert torch.equal(x, y)

    lengths = torch.tensor([n * sbs, 5 * sbs - 7], device=device) if use_causal else None
    cache = {}
    mask = new_mask(1)
    first = run(mask, lengths, cache)
    facts = cache["mask_facts"].cache["facts"]
    assert facts.group_offsets is None and facts.bwd_scratch is not None
    same(run(mask, lengths, cache), first)
    assert cache["mask_facts"].cache["facts"] is facts and facts.group_offsets is not None
    assert int(facts.group_offsets[-1]) < int(cache["group_offsets"][-1])
    same(run(mask, lengths, cache), first)
    same(run(mask, lengths, {}), first)

    mask[::2] = False  # in place: the version counter moves
    changed = run(mask, lengths, cache)
    assert cache["mask_facts"].cache["facts"] is not facts
    fresh = run(mask, lengths, {})
    assert not torch.equal(changed[0], first[0])
    same(changed, fresh)
    same(run(mask, lengths, cache), fresh)
    same(run(mask, lengths, cache), fresh)

    other = new_mask(2)
    same(run(other, lengths, cache), run(other, lengths, {}))
    same(run(other, lengths, cache), run(other, lengths, {}))
    if use_causal:
        shorter = torch.tensor([3 * sbs + 1, n * sbs], device=device)
        same(run(other, shorter, cache), run(other, shorter, {}))
        same(run(other, shorter, cache), run(other, shorter, {}))
        shorter[0] = 2 * sbs  # in place
        same(run(other, shorter, cache), run(other, shorter, {}))

    # against the oracle, with the lists of the second sighting
    ref_q, ref_k, ref_v = (t.cpu().double().requires_grad_(True) for t in (q, k, v))
    ref = orc.flash_attention(ref_q, full.cpu().numpy(), ref_k, full.cpu().numpy(), ref_v, full.cpu().numpy(),
                              la.cpu().numpy(), sbs, mask=other.cpu(), layout_mask=lmask.cpu().numpy(),
                              causal_lengths=None if lengths is None else lengths.cpu(), acc_dtype=torch.float64)
    ref.backward(go.cpu().double())
    run(other, lengths, cache)
    got = run(other, lengths, cache)
    assert_close(got[0], ref, 2e-2, "O")
    for name, a, b in (("dQ", got[1], ref_q.grad), ("dK", got[2], ref_k.grad), ("dV", got[3], ref_v.grad)):
        assert_close(a, b, 2e-2, name)


def test_dead_pairs_listed_at_the_first_sighting_on_a_large_layout(device, monkeypatch):
    """From a threshold of active blocks on, the forward lists without dead pairs are built at the first call with
    a mask (here the threshold is lowered to the test's size): same bits as with lists built at the second call,
    forward and backward, and the first call already walks the shorter lists."""
    import sys
    fa = sys.modules["blksprs_amd.ops.flash_attention"]  # the package attribute of that name is the function
    g = torch.Generator().manual_seed(31)
    B, n, nh, sbs = 2, 8, 2, 64
    la = orc.random_layout((B, n, n), 0.7, g, ensure_rows=True).to(device)
    full = torch.ones((B, n, nh), dtype=torch.bool, device=device)
    q, k, v = (rand_blocks(B * n * nh, sbs, torch.bfloat16, s).to(device) for s in (1, 2, 3))
    go = rand_blocks(B * n * nh, sbs, torch.bfloat16, 4).to(device)
    n_mask = int(la.sum())
    gm = torch.Generator().manual_seed(5)
    mask = torch.rand((n_mask, sbs, sbs), generator=gm) < 0.3
    mask[torch.rand(n_mask, generator=gm) < 0.5] = True  # dead pairs
    mask = mask.to(device)

    def run(cache):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = bs.ops.flash_attention(qq, full, kk, full, vv, full, la, sbs, attention_mask=mask,
                                     sparsity_layout_mask=la, layout_cache=cache)
        out.backward(go)
        return out.detach(), qq.grad, kk.grad, vv.grad

    late = {}
    reference = run(late)
    assert late["mask_facts"].cache["facts"].group_offsets is None
    monkeypatch.setattr(fa, "_PRUNE_AT_ONCE_BLOCKS", 1)
    early = {}
    first = run(early)
    facts = early["mask_facts"].cache["facts"]
    assert facts.group_offsets is not None and int(facts.group_offsets[-1]) < int(early["group_offsets"][-1])
    for a, b in zip(first, reference):
        assert torch.equal(a, b)
    for a, b in zip(run(early), reference):
        assert torch.equal(a, b)
    assert early["mask_facts"].cache["facts"] is facts


def test_a_mask_that_masks_everything_leaves_empty_lists(device):
    """Every mask block masks everything: from the second call on the forward's lists are empty.  Output and
    gradients are zeros, as on the first call."""
    B, n, nh, sbs = 1, 4, 1, 64
    la = torch.ones((B, n, n), dtype=torch.bool, device=device)
    full = torch.ones((B, n, nh), dtype=torch.bool, device=device)
    q, k, v = (rand_blocks(B * n * nh, sbs, torch.bfloat16, s).to(device) for s in (1, 2, 3))
    mask = torch.ones((B * n * n, sbs, sbs), dtype=torch.bool, device=device)
    cache = {}
    results = []
    for _ in range(3):
        qq = q.clone().requires_grad_(True)
        out = bs.ops.flash_attention(qq, full, k, full, v, full, la, sbs, attention_mask=mask,
                                     sparsity_layout_mask=la, layout_cache=cache)
        out.sum().backward()
        results.append((out.detach(), qq.grad))
    facts = cache["mask_facts"].cache["facts"]
    assert facts.group_offsets is not None and int(facts.group_offsets[-1]) == 0
    for out, grad in results:
        assert torch.all(out == 0) and torch.all(grad == 0)


def test_lists_kept_per_causal_lengths(device):
    """Native causal attention without a mask tensor: from the second call with one tensor of lengths on, the
    forward walks lists without the pairs the causal predicate rules out as a whole.  Same bits as the first
    call and as a fresh cache; lengths changed in place give what a fresh cache gives."""
    g = torch.Generator().manual_seed(22)
    B, n, nh, sbs = 2, 8, 2, 64
    la = orc.random_layout((B, n, n), 0.8, g, ensure_rows=True).to(device)
    full = torch.ones((B, n, nh), dtype=torch.bool, device=device)
    q, k, v = (rand_blocks(B * n * nh, sbs, torch.bfloat16, s).to(device) for s in (1, 2, 3))
    go = rand_blocks(B * n * nh, sbs, torch.bfloat16, 4).to(device)
    lengths = torch.tensor([n * sbs, 5 * sbs - 9], device=device)

    def run(cache):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = bs.ops.flash_attention(qq, full, kk, full, vv, full, la, sbs, layout_cache=cache,
                                     causal_lengths=lengths)
        out.backward(go)
        return out.detach(), qq.grad, kk.grad, vv.grad

    cache = {}
    first = run(cache)
    for _ in range(2):
        for a, b in zip(run(cache), first):
            assert torch.equal(a, b)
    facts = cache["mask_facts"].cache["facts"]
    assert int(facts.group_offsets[-1]) < int(cache["group_offsets"][-1])
    lengths[1] = 2 * sbs + 1
    changed, fresh = run(cache), run({})
    assert not torch.equal(changed[0], first[0])
    for a, b in zip(changed, fresh):
        assert torch.equal(a, b)
    for a, b in zip(run(cache), fresh):
        assert torch.equal(a, b)
    ref_q, ref_k, ref_v = (t.cpu().double().requires_grad_(True) for t in (q, k, v))
    ref = orc.flash_attention(ref_q, full.cpu().numpy(), ref_k, full.cpu().numpy(), ref_v, full.cpu().numpy(),
                              la.cpu().numpy(), sbs, causal_lengths=lengths.cpu(), acc_dtype=torch.float64)
    ref.backward(go.cpu().double())
    got = run(cache)
    assert_close(got[0], ref, 2e-2, "O")
    for name, a, b in (("dQ", got[1], ref_q.grad), ("dK", got[2], ref_k.grad), ("dV", got[3], ref_v.grad)):
        assert_close(a, b, 2e-2, name)
