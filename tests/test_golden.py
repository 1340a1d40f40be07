"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): fixed inputs with the
outputs the CPU oracle gave for them when the files were committed.  The CPU tests hold the oracle to the
files; the GPU tests hold the HIP path to them (bit-exact for the integer tables, 1e-5 for fp32)."""

from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import blksprs_oracle as orc
from tests.helpers import assert_close

GOLDEN = Path(__file__).resolve().parent / "golden"


def _load(name):
    return dict(np.load(GOLDEN / name, allow_pickle=False))


def test_oracle_reproduces_the_lookup_table_fixture():
    d = _load("lut.npz")
    lx, ly, lo = d["layout_x"], d["layout_y"], d["layout_o"]
    assert np.array_equal(orc.layout_matmul(lx, ly), lo)
    assert np.array_equal(orc.packed_indices(lx), d["packed_x"])
    assert np.array_equal(orc.layout_indices(lo), d["nonzero_o"])
    off, pairs = orc.contraction_lists(lx, ly, lo)
    assert np.array_equal(off, d["pair_offsets"]) and np.array_equal(pairs, d["pairs"])
    idx, offsets, longest = orc.segmented_indices(lx)
    assert np.array_equal(idx, d["csr_indices"]) and np.array_equal(offsets, d["csr_offsets"])
    assert longest == int(d["csr_longest"])
    srt, mbl = orc.sorted_packed_indices(lx)
    assert np.array_equal(srt, d["sorted_rows"]) and mbl == int(d["max_blocks_line"])


def test_oracle_reproduces_the_compute_fixture():
    d = _load("compute.npz")
    sbs = int(d["sbs"])
    t = lambda k: torch.from_numpy(d[k])
    mm = orc.matmul(t("x"), d["layout_x"], t("y"), d["layout_y"], d["layout_o"], sbs, acc_dtype=torch.float64)
    assert_close(mm, t("matmul"), 1e-12, "matmul")
    assert_close(orc.softmax(t("softmax_in"), d["layout_x"], sbs), t("softmax"), 1e-12, "softmax")
    B, nq, nk = d["attention_layout"].shape
    at = orc.flash_attention(t("q"), np.ones((B, nq, 1), bool), t("k"), np.ones((B, nk, 1), bool), t("v"),
                             np.ones((B, nk, 1), bool), d["attention_layout"], sbs, mask=t("mask"),
                             layout_mask=d["layout_mask"], acc_dtype=torch.float64)
    assert_close(at, t("attention"), 1e-12, "attention")


@pytest.mark.gpu
def test_device_lookup_tables_match_the_fixture(device):
    from blksprs_amd.ops.flash_attention import _build_segmented_indices
    from blksprs_amd.ops.matmul import matmul_build_layout_cache
    from blksprs_amd.ops.softmax import softmax_fused_build_layout_cache
    import blksprs_amd as bs
    d = _load("lut.npz")
    lx, ly = (torch.from_numpy(d[k]).to(device) for k in ("layout_x", "layout_y"))
    lo = bs.layouting.build_sparsity_layout_matmul(lx, ly)
    assert np.array_equal(lo.cpu().numpy() != 0, d["layout_o"])
    cache = matmul_build_layout_cache(None, lx, ly, lo)
    assert np.array_equal(cache["packed_indices_x"].cpu().numpy(), d["packed_x"])
    assert np.array_equal(cache["layout_indices_o"].cpu().numpy(), d["nonzero_o"])
    assert np.array_equal(cache["contraction_offsets"].cpu().numpy(), d["pair_offsets"])
    assert np.array_equal(cache["contraction_pairs"].cpu().numpy(), d["pairs"])
    B, R, C = d["layout_x"].shape
    idx, off, longest = _build_segmented_indices(lx, B, R, C)
    assert np.array_equal(idx.cpu().numpy(), d["csr_indices"]) and np.array_equal(off.cpu().numpy(), d["csr_offsets"])
    assert longest == int(d["csr_longest"])
    sm = softmax_fused_build_layout_cache(None, lx)
    assert np.array_equal(sm["packed_indices_sorted"].cpu().numpy().reshape(-1), d["sorted_rows"])
    assert sm["max_blocks_line"] == int(d["max_blocks_line"])


@pytest.mark.gpu
def test_device_results_match_the_compute_fixture(device):
    import blksprs_amd as bs
    d = _load("compute.npz")
    sbs = int(d["sbs"])
    f32 = lambda k: torch.from_numpy(d[k]).float().to(device)
    lay = lambda k: torch.from_numpy(d[k]).to(device)
    out = bs.ops.matmul(f32("x"), lay("layout_x"), f32("y"), lay("layout_y"), lay("layout_o"), sbs)
    assert_close(out, torch.from_numpy(d["matmul"]), 1e-5, "matmul fp32")
    out = bs.ops.softmax(f32("softmax_in"), lay("layout_x"), sbs)
    assert_close(out, torch.from_numpy(d["softmax"]), 1e-5, "softmax fp32")
    B, nq, nk = d["attention_layout"].shape
    ones = lambda n: torch.ones((B, n, 1), dtype=torch.bool, device=device)
    out = bs.ops.flash_attention(f32("q"), ones(nq), f32("k"), ones(nk), f32("v"), ones(nk), lay("attention_layout"),
                                 sbs, attention_mask=lay("mask"), sparsity_layout_mask=lay("layout_mask"))
    assert_close(out, torch.from_numpy(d["attention"]), 2e-5, "attention fp32")


def test_oracle_reproduces_the_neighbours_fixture():
    d = _load("neighbours.npz")
    sbs = int(d["sbs"])
    t = lambda k: torch.from_numpy(d[k])
    layout = d["layout"]
    xt, layout_t = orc.transpose(t("x"), layout, sbs)
    assert torch.equal(xt, t("transposed")) and np.array_equal(layout_t, d["layout_t"])
    assert np.array_equal(orc.build_sparsity_layout(orc.to_dense(t("x"), layout, sbs), sbs), d["dense_layout"])
    row_sum, row_layout = orc.row_wise_reduce(t("x"), layout, sbs, "sum")
    assert np.array_equal(row_layout, d["row_layout"])
    assert_close(row_sum, t("row_sum"), 1e-12, "row sum")
    row_max, _ = orc.row_wise_reduce(t("x"), layout, sbs, "max", slice_only=True)
    assert torch.equal(row_max, t("row_max"))
    assert torch.equal(orc.row_wise_add(t("x"), layout, -row_max, sbs), t("centred"))
    lin, lin_layout = orc.linear(t("x"), layout, t("weight"), t("bias"), sbs)
    assert np.array_equal(lin_layout, d["linear_layout"])
    assert_close(lin, t("linear"), 1e-12, "linear")
    lengths = d["lengths"]
    assert np.array_equal(orc.causal_layout(lengths, sbs), d["causal_layout"])
    assert np.array_equal(orc.causal_layout(lengths, sbs, window_size=23), d["window_layout"])
    assert np.array_equal(orc.causal_mask_layout(lengths, d["causal_layout"], sbs), d["causal_mask_layout"])
    assert np.array_equal(orc.causal_mask_layout(lengths, d["window_layout"], sbs, window_size=23),
                          d["window_mask_layout"])


@pytest.mark.gpu
def test_device_results_match_the_neighbours_fixture(device):
    import blksprs_amd as bs
    d = _load("neighbours.npz")
    sbs = int(d["sbs"])
    f32 = lambda k: torch.from_numpy(d[k]).float().to(device)
    lay = lambda k: torch.from_numpy(d[k]).to(device)
    x, layout = bs.BlksprsTensor.wrap(f32("x")), lay("layout")
    xt, layout_t = bs.ops.transpose(x, layout, sbs)
    assert torch.equal(xt.cpu(), torch.from_numpy(d["transposed"]).float())
    assert np.array_equal(layout_t.cpu().numpy() != 0, d["layout_t"])
    dense = bs.ops.to_dense(x, layout, sbs)
    assert np.array_equal(bs.layouting.build_sparsity_layout(dense, sbs).cpu().numpy() != 0, d["dense_layout"])
    row_sum, row_layout = bs.ops.misc.row_wise_sum(x, layout, sbs)
    assert np.array_equal(row_layout.cpu().numpy() != 0, d["row_layout"])
    assert_close(row_sum, torch.from_numpy(d["row_sum"]), 1e-5, "row sum fp32")
    row_max, _ = bs.ops.misc.row_wise_max(x, layout, sbs, flag_slice_only=True)
    assert torch.equal(row_max.cpu(), torch.from_numpy(d["row_max"]).float())
    centred = bs.ops.misc.row_wise_sub(x, layout, row_max, sbs)
    assert_close(centred, torch.from_numpy(d["centred"]), 1e-6, "x - row max")
    linear = torch.nn.Linear(d["weight"].shape[1], d["weight"].shape[0], device=device)
    with torch.no_grad():
        linear.weight.copy_(f32("weight"))
        linear.bias.copy_(f32("bias"))
    lin, lin_layout = bs.utils.apply_torch_linear(x, layout, sbs, linear)
    assert np.array_equal(lin_layout.cpu().numpy() != 0, d["linear_layout"])
    assert_close(lin, torch.from_numpy(d["linear"]), 1e-5, "linear fp32")
    lengths = lay("lengths")
    causal = bs.layouting.build_causal_self_attention_layout(lengths, sbs)
    window = bs.layouting.build_causal_window_self_attention_layout(lengths, sbs, 23)
    assert np.array_equal(causal.cpu().numpy() != 0, d["causal_layout"])
    assert np.array_equal(window.cpu().numpy() != 0, d["window_layout"])
    _, mask_layout = bs.layouting.build_causal_self_attention_mask(lengths, causal, sbs)
    assert np.array_equal(mask_layout.cpu().numpy() != 0, d["causal_mask_layout"])
    _, mask_layout = bs.layouting.build_causal_window_self_attention_mask(lengths, window, sbs, 23)
    assert np.array_equal(mask_layout.cpu().numpy() != 0, d["window_mask_layout"])
