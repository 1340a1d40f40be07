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
