"""Host-side behaviour that needs no GPU: validation switches and messages, the layout cache rules, the
shape helpers, and that the operators refuse CPU tensors instead of computing somewhere else."""

import threading

import pytest
import torch

import blksprs_amd as bs
from blksprs_amd.utils import tools, validation


def test_public_surface():
    for name in ("matmul", "flash_attention", "flash_attention_build_layout_cache", "softmax", "softmax_fused",
                 "to_sparse", "to_dense", "to_blksprs", "from_blksprs", "to_sparse_shaped", "to_dense_shaped"):
        assert callable(getattr(bs.ops, name))
    assert callable(bs.layouting.build_sparsity_layout_matmul)
    for name in ("disable_validation", "enable_validation", "disable_contiguous", "enable_contiguous",
                 "do_shape_blocksparse", "undo_shape_blocksparse"):
        assert callable(getattr(bs.utils, name))


def test_blksprs_tensor_wrap():
    t = torch.zeros((1, 16, 16))
    w = bs.BlksprsTensor.wrap(t)
    assert isinstance(w, bs.BlksprsTensor) and w.data_ptr() == t.data_ptr()
    assert repr(w).startswith("BlksprsTensor(tensor(")
    assert type(tools.as_base_tensor(w)) is torch.Tensor


def test_operators_refuse_cpu_tensors():
    lay = torch.ones((1, 1, 1), dtype=torch.bool)
    x = torch.zeros((1, 16, 16))
    with pytest.raises(ValueError, match="Tensors must be on GPU"):
        bs.ops.matmul(x, lay, x, lay, lay, 16)
    with pytest.raises(ValueError, match="Tensors must be on GPU"):
        bs.ops.softmax(x, lay, 16)
    with pytest.raises(ValueError, match="Tensors must be on GPU"):
        bs.ops.to_dense(x, lay, 16)
    with pytest.raises(ValueError, match="Tensors must be on GPU"):
        bs.ops.flash_attention(x, lay, x, lay, x, lay, lay, 16)
    # with validation off there is still no CPU path: the LUT builder itself refuses
    bs.utils.disable_validation()
    try:
        with pytest.raises(RuntimeError, match="needs GPU tensors"):
            bs.ops.to_dense(x, torch.ones((1, 2, 1), dtype=torch.bool), 16)
    finally:
        bs.utils.enable_validation()


def test_validation_messages():
    v = validation
    with pytest.raises(ValueError, match="Tensor must have 3 dimensions"):
        v.validate_dimensions(torch.zeros(2, 2))
    with pytest.raises(ValueError, match="Tensor must be contiguous"):
        v.validate_contiguous(torch.zeros(4, 4).t())
    with pytest.raises(ValueError, match="either float16, bfloat16, or float32"):
        v.validate_dtype_float(torch.zeros(1, dtype=torch.float64))
    with pytest.raises(ValueError, match="same dtype"):
        v.validate_dtype_float(torch.zeros(1), torch.zeros(1, dtype=torch.float16))
    with pytest.raises(ValueError, match="float32 dtype"):
        v.validate_dtype_float_32(torch.zeros(1, dtype=torch.float16))
    with pytest.raises(ValueError, match="0 or 1"):
        v.validate_binary(torch.tensor([0.0, 2.0]))
    with pytest.raises(TypeError, match="must be an integer"):
        v.validate_sparsity_block_size(True)
    with pytest.raises(TypeError, match="must be an integer"):
        v.validate_sparsity_block_size(16.0)
    with pytest.raises(ValueError, match="at least 16"):
        v.validate_sparsity_block_size(8)
    with pytest.raises(ValueError, match="power of 2"):
        v.validate_sparsity_block_size(48)
    with pytest.raises(ValueError, match="divisible by sparsity block size"):
        v.validate_sparsity_block_size(32, torch.zeros(1, 48, 32))
    with pytest.raises(ValueError, match=r"Output sparsity layout shape \(1, 2\) doesn't match expected \(2, 1\)"):
        v.validate_shape(torch.zeros(1, 2), (2, 1), "Output sparsity layout")
    with pytest.raises(ValueError, match="complex dtype"):
        v.validate_sparsity(16, (torch.zeros(1, 16, 16), torch.ones((1, 1, 1), dtype=torch.complex64)))
    with pytest.raises(ValueError, match="Blocks not conforming"):
        v.validate_sparsity(16, (torch.zeros(1, 16, 32), torch.ones((1, 1, 1))))
    with pytest.raises(ValueError, match="Mismatch between sparsity layout and blocks"):
        v.validate_sparsity(16, (torch.zeros(2, 16, 16), torch.ones((1, 1, 1))))
    with pytest.raises(ValueError, match="exactly 3 dimensions"):
        v.validate_sparsity(16, (torch.zeros(1, 16, 16), torch.ones((1, 1))))
    with pytest.raises(TypeError, match="must be an integer"):
        v.validate_positive_integer(1.5, "Repeats")
    with pytest.raises(ValueError, match="positive integer"):
        v.validate_positive_integer(0, "Repeats")


def test_switches_are_per_thread():
    bs.utils.disable_validation()
    bs.utils.disable_contiguous()
    seen = {}

    def worker():
        seen["validation"] = validation._validation_enabled()
        seen["contiguous"] = validation._contiguous_enabled()

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    try:
        assert seen == {"validation": True, "contiguous": True}
        assert not validation._validation_enabled()
        validation.validate_dimensions(torch.zeros(2))  # no-op while disabled
        nc = torch.zeros(4, 4).t()
        assert validation.ensure_contiguous(nc) is nc
    finally:
        bs.utils.enable_validation()
        bs.utils.enable_contiguous()
    assert validation.ensure_contiguous(torch.zeros(4, 4).t()).is_contiguous()


def test_layout_cache_rules():
    lay = torch.ones((1, 2, 2), dtype=torch.bool)
    cache = tools.prepare_layout_cache(None, "op", lay, 3)
    cache["table"] = torch.arange(4)
    cache["count"] = 4
    tools.finalize_layout_cache(cache)
    assert tools.prepare_layout_cache(cache, "op", lay, 3).get("count") == 4      # hit
    assert "count" not in tools.prepare_layout_cache(cache, "other", lay, 3)       # other operation
    cache["count"] = 4
    tools.finalize_layout_cache(cache)
    assert "count" not in tools.prepare_layout_cache(cache, "other", lay, 4)       # other scalar
    cache["count"] = 4
    tools.finalize_layout_cache(cache)
    lay[0, 0, 0] = False                                                            # source mutated in place
    assert "count" not in tools.prepare_layout_cache(cache, "other", lay, 4)
    cache["table"] = torch.arange(4)
    tools.finalize_layout_cache(cache)
    cache["table"].add_(1)                                                          # derived entry mutated
    assert "table" not in tools.prepare_layout_cache(cache, "other", lay, 4)
    cache["x"] = 1                                                                  # never finalized
    assert "x" not in tools.prepare_layout_cache(cache, "other", lay, 4)
    # sources are retained so their ids cannot be recycled
    assert cache["_blksprs_cache_refs"][0] is lay
    with torch.inference_mode():
        inf = torch.ones((1, 1, 1))
    c2 = tools.prepare_layout_cache(None, "op", inf)
    c2["v"] = 1
    tools.finalize_layout_cache(c2)
    assert "v" not in tools.prepare_layout_cache(c2, "op", inf)                     # inference tensors never hit


def test_shape_helpers():
    x = torch.zeros((2, 3, 4, 5))
    flat, shape = tools.do_shape_blocksparse(x)
    assert flat.shape == (6, 4, 5) and shape == x.shape
    assert tools.undo_shape_blocksparse(flat, shape).shape == x.shape
    assert tools.undo_shape_blocksparse(torch.zeros((6, 4, 7)), shape).shape == (2, 3, 4, 7)
    with pytest.raises(ValueError, match="at least 2 dimensions"):
        tools.do_shape_blocksparse(torch.zeros(3))
    with pytest.raises(ValueError, match="batch dimension does not match"):
        tools.undo_shape_blocksparse(torch.zeros((5, 4, 5)), shape)
    assert tools.ceil_pow2(1) == 1 and tools.ceil_pow2(5) == 8 and tools.ceil_pow2(8) == 8
    with pytest.raises(ValueError):
        tools.ceil_pow2(0)
    assert tools.can_use_int32_indexing(torch.zeros(4), None, 2_147_483_647)
    assert not tools.can_use_int32_indexing(2_147_483_648)


def test_unknown_autotune_mode_is_rejected():
    import os
    import subprocess
    import sys
    env = dict(os.environ, BLKSPRS_AUTOTUNE="FAST")
    proc = subprocess.run([sys.executable, "-c", "import blksprs_amd"], env=env, capture_output=True, text=True,
                          cwd=str(__import__("pathlib").Path(__file__).resolve().parent.parent))
    assert proc.returncode != 0 and "Unknown autotune mode" in proc.stderr


def test_row_work_table_holds_every_part_once_and_keeps_eighths_together():
    """The table of the row kernel: entries row << parts_log2 | part, the k-th item of the c-th contiguous
    eighth of the rows at position 8 k + c, -1 where an eighth has a row less; inside an eighth batch entries
    ascend, parts ascend inside an entry, and inside a part the rows with the most pairs come first.  Checked
    here on the restatement in torch that the device builder is held to bit for bit (test_lut_gpu.py)."""
    import importlib
    from types import SimpleNamespace
    from tests import helpers
    real = importlib.import_module("blksprs_amd.ops.matmul")
    mm = SimpleNamespace(_row_work_table=helpers.expected_row_work_table, _ROWS_DOWNWARD=helpers.ROWS_DOWNWARD,
                         _row_parts_log2=real._row_parts_log2)
    g = torch.Generator().manual_seed(5)
    for n_rows, rows_per_batch, parts_log2 in ((1024, 64, 0), (1024, 64, 1), (21, 7, 2), (5, 5, 1), (8, 1, 3)):
        blocks_per_row = 9
        row_offsets = torch.arange(n_rows + 1, dtype=torch.int32) * blocks_per_row
        pair_offsets = torch.cumsum(torch.randint(0, 6, (n_rows * blocks_per_row + 1,), generator=g), 0).to(torch.int32)
        work = (pair_offsets[row_offsets.long()][1:] - pair_offsets[row_offsets.long()][:-1]).tolist()
        table = mm._row_work_table(pair_offsets, row_offsets, rows_per_batch, parts_log2)
        # a bound on a row's pairs that the caller knows in advance gives the same table as the measured maximum
        assert torch.equal(table, mm._row_work_table(pair_offsets, row_offsets, rows_per_batch, parts_log2,
                                                     max_work=5 * blocks_per_row + 100))
        # with a sweep every second run of `sweep` items of a (XCD, batch entry, part) group carries the downward flag
        swept = mm._row_work_table(pair_offsets, row_offsets, rows_per_batch, parts_log2, sweep=3)
        assert torch.equal(torch.where(swept >= 0, swept & ~mm._ROWS_DOWNWARD, swept), table)
        for c in range(8):
            run, last_group = 0, None
            for e in swept[c::8].tolist():
                if e < 0:
                    continue
                plain = e & ~mm._ROWS_DOWNWARD
                group = ((plain >> parts_log2) // rows_per_batch, plain & ((1 << parts_log2) - 1))
                run = run + 1 if group == last_group else 0
                last_group = group
                assert bool(e & mm._ROWS_DOWNWARD) == bool((run // 3) & 1)
        parts = 1 << parts_log2
        assert table.dtype == torch.int32 and table.numel() % 8 == 0
        live = table[table >= 0].long()
        assert torch.equal(torch.sort(live)[0], torch.arange(n_rows * parts))
        assert table.numel() == -(-n_rows // 8) * parts * 8
        small, extra = divmod(n_rows, 8)
        start = 0
        for c in range(8):
            size = small + (c < extra)
            items = [int(e) for e in table[c::8].tolist()]
            assert all(e == -1 for e in items[size * parts:])
            items = items[:size * parts]
            rows = [e >> parts_log2 for e in items]
            assert sorted(set(rows)) == list(range(start, start + size))
            order = [(r // rows_per_batch, e & (parts - 1), -work[r]) for e, r in zip(items, rows)]
            assert order == sorted(order)
            start += size
    assert mm._row_work_table(torch.zeros(1, dtype=torch.int32), torch.zeros(1, dtype=torch.int32), 1, 1).numel() == 0
    # two parts only when an entry's y blocks are several times one L2 and the rows are long enough to feed the
    # waves twice
    assert mm._row_parts_log2(1024, 64, 64, 16287, 64370, 8192) == 0      # configuration 2: 8 MB per entry
    assert mm._row_parts_log2(1024, 64, 64, 4 * 16287, 64370, 8192) == 1  # 32 MB per entry
    assert mm._row_parts_log2(1024, 64, 64, 4 * 16287, 16000, 8192) == 0  # short rows
    # with pair_up a group's rows alternate longest, shortest, second longest, second shortest, ...: 16 rows of one
    # batch entry, two per XCD, the work ascending with the row: every XCD's list is (its longer row, its shorter)
    ascending = torch.cumsum(torch.arange(17, dtype=torch.int32) * 3, 0).to(torch.int32)
    paired = mm._row_work_table(ascending, torch.arange(17, dtype=torch.int32), 16, 0, pair_up=True)
    plain = mm._row_work_table(ascending, torch.arange(17, dtype=torch.int32), 16, 0)
    for c in range(8):
        assert paired[c::8].tolist() == [2 * c + 1, 2 * c] == plain[c::8].tolist()
    # one XCD list of 5 rows (40 rows, one batch entry): longest, shortest, second longest, second shortest, middle
    offsets = torch.cumsum(torch.arange(41, dtype=torch.int32), 0).to(torch.int32)
    paired = mm._row_work_table(offsets, torch.arange(41, dtype=torch.int32), 40, 0, pair_up=True)
    assert paired[0::8].tolist() == [4, 0, 3, 1, 2]


def test_the_limit_on_kept_ds_is_a_process_wide_setting():
    """``bs.utils.set_kept_ds_limit`` is what ``flash_attention``'s backward asks (through ``kept_ds_limit``) before it
    requests room for dS; 0 turns the kept dS off."""
    import blksprs_amd as bs
    from blksprs_amd.utils import validation
    before = validation.kept_ds_limit()
    try:
        assert before == 4 << 30
        bs.utils.set_kept_ds_limit(0)
        assert validation.kept_ds_limit() == 0
        bs.utils.set_kept_ds_limit(1 << 20)
        assert validation.kept_ds_limit() == 1 << 20
    finally:
        bs.utils.set_kept_ds_limit(before)


def test_measurement_knobs_are_clamped_and_malformed_values_ignored(monkeypatch):
    """The environment variables that steer the row kernel's work order for measurements are clamped to their legal
    range, and a value that is no integer is ignored with a warning instead of failing every product."""
    import importlib
    import warnings
    mm = importlib.import_module("blksprs_amd.ops.matmul")
    monkeypatch.setenv("BLKSPRS_AMD_ROW_PARTS_LOG2", "-1")
    assert mm._measurement_knob("BLKSPRS_AMD_ROW_PARTS_LOG2", 1, 0, 3) == 0
    monkeypatch.setenv("BLKSPRS_AMD_ROW_PARTS_LOG2", "9")
    assert mm._measurement_knob("BLKSPRS_AMD_ROW_PARTS_LOG2", 1, 0, 3) == 3
    assert mm._row_parts_log2(1024, 64, 64, 16384, 64512, 8192) == 3
    monkeypatch.setenv("BLKSPRS_AMD_ROW_PARTS_LOG2", "two")
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        assert mm._measurement_knob("BLKSPRS_AMD_ROW_PARTS_LOG2", 1, 0, 3) == 1
    assert any("not an integer" in str(w.message) for w in caught)
    monkeypatch.delenv("BLKSPRS_AMD_ROW_PARTS_LOG2")
    assert mm._measurement_knob("BLKSPRS_AMD_ROW_PARTS_LOG2", 1, 0, 3) == 1


def test_line_kernel_is_chosen_within_its_limits_only():
    """The backward products take the line kernel for 16-bit operands at sbs 64 when no line of either layout has
    more than 512 blocks and there are fewer than 2^25 lines (the part table holds the line in 25 bits and
    bsa_matmul_lines_parts refuses more); everything else takes the tile kernel."""
    import importlib
    mm = importlib.import_module("blksprs_amd.ops.matmul")
    ok = lambda B, R, K, C, sbs=64, dt=torch.bfloat16: mm._lines_apply(None, ((B, R, K), (B, K, C)), sbs, dt)
    assert ok(16, 64, 64, 64) and ok(1, 512, 512, 512) and ok(2, 4, 6, 5, dt=torch.float16)
    assert not ok(16, 64, 64, 64, sbs=32) and not ok(16, 64, 64, 64, dt=torch.float32)
    assert not ok(1, 513, 8, 8) and not ok(1, 8, 513, 8) and not ok(1, 8, 8, 513)
    assert ok((1 << 25) // 512 - 1, 512, 8, 8) and not ok((1 << 25) // 512, 512, 8, 8)
    assert not ok((1 << 25) // 512, 8, 8, 512)
