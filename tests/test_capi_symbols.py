"""The C-ABI library loads and exports exactly what include/blksprs_amd.h declares (no compute calls)."""

import ctypes
import re
from pathlib import Path

from blksprs_amd import _capi

HEADER = Path(__file__).resolve().parent.parent / "include" / "blksprs_amd.h"


def _declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(bsa_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_entry_points():
    assert _declared() == sorted(_capi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(_capi.library_path()))
    for name in _declared():
        assert hasattr(lib, name), name
    assert _capi.load().bsa_abi_version() == _capi.ABI_VERSION


def test_library_names_the_compiler_it_was_built_with():
    # the hand-placed waits of some kernels were found with one compiler: a changed toolchain shows here, next to
    # whatever bit-identity test it may turn red
    info = _capi.load().bsa_build_info().decode()
    print("\n" + info)
    assert info.startswith("hipcc: ") and "flags:" in info and "unknown" not in info


def test_argument_block_matches_the_header_layout():
    # 24 pointers, 11 int64, 3 int32 and one float, then 2 pointers and one int32 (padded to 8 bytes), a pointer
    # and three int64, a pointer and an int64
    assert ctypes.sizeof(_capi.AttnArgs) == 24 * 8 + 11 * 8 + 4 * 4 + 2 * 8 + 8 + 4 * 8 + 2 * 8
    assert _capi.AttnArgs.bwd_ds.offset == 44 * 8 and _capi.AttnArgs.bwd_ds_bytes.offset == 45 * 8
    assert _capi.AttnArgs.bwd_scratch.offset == 40 * 8 and _capi.AttnArgs.n_layout_blocks.offset == 41 * 8
    assert _capi.AttnArgs.bwd_scratch_ready.offset == 42 * 8 and _capi.AttnArgs.bwd_scratch_bytes.offset == 43 * 8
    assert _capi.AttnArgs.group_offsets.offset == 37 * 8 and _capi.AttnArgs.group_size.offset == 39 * 8
    assert _capi.AttnArgs.sbs.offset == 35 * 8


def test_bad_arguments_are_rejected_on_the_host():
    lib = _capi.load()
    # sbs = 24 is not a power of two; nothing is launched
    rc = lib.bsa_matmul(0, 0, 0, 0, 0, 0, 0, 0, 0, 24, 0, 0, 0, 0)
    assert rc == -1 and b"power of two" in lib.bsa_last_error()
    rc = lib.bsa_to_sparse(0, 0, 0, 0, 32, 32, 16, 3, 0)
    assert rc == -1 and b"element size" in lib.bsa_last_error()
    # empty problems are accepted without touching the device
    assert lib.bsa_matmul(0, 0, 0, 0, 0, 0, 0, 0, 0, 64, 2, 0, 0, 0) == 0
    assert lib.bsa_softmax_fwd(0, 0, 0, 0, 0, 32, 0) == 0


def test_bad_arguments_of_the_neighbouring_entry_points_are_rejected_on_the_host():
    lib = _capi.load()
    F32, BF16 = _capi.F32, _capi.BF16
    # row-wise reduction: unknown operation, unknown dtype, block size not a power of two
    assert lib.bsa_row_reduce(0, 0, 0, 0, 1, 1, 1, 64, F32, 2, 0, 0) == -1 and b"op must be" in lib.bsa_last_error()
    assert lib.bsa_row_reduce(0, 0, 0, 0, 1, 1, 1, 64, 99, 0, 0, 0) == -1 and b"dtype" in lib.bsa_last_error()
    assert lib.bsa_row_reduce(0, 0, 0, 0, 1, 1, 1, 48, F32, 0, 0, 0) == -1 and b"power of two" in lib.bsa_last_error()
    assert lib.bsa_row_reduce(0, 0, 0, 0, 0, 0, 0, 64, BF16, 1, 1, 0) == 0  # nothing to do
    # row-wise add: y has 1 or sbs columns
    assert lib.bsa_row_add(0, 0, 0, 0, 0, 1, 1, 1, 1, 2, 64, F32, 0) == -1 and b"1 or sbs columns" in lib.bsa_last_error()
    assert lib.bsa_row_add(0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 64, F32, 0) == 0
    # transpose and layout of a dense tensor: element size, and a 1-byte floating-point type does not exist
    assert lib.bsa_transpose_blocks(0, 0, 0, 0, 1, 1, 1, 1, 1, 64, 3, 0) == -1 and b"element size" in lib.bsa_last_error()
    assert lib.bsa_transpose_blocks(0, 0, 0, 0, 0, 0, 1, 1, 1, 64, 2, 0) == 0
    assert lib.bsa_layout_from_dense(0, 0, 1, 1, 1, 64, 1, 1, 0) == -1 and b"1 byte" in lib.bsa_last_error()
    assert lib.bsa_layout_from_dense(0, 0, 0, 1, 1, 64, 2, 1, 0) == 0
    # scratch of the attention backward: 2 x 32 bytes per layout block, (4 + 64) per row, 64 bytes of tickets, one
    # byte per mask block
    assert lib.bsa_attn_bwd_scratch_bytes(2, 3, 5, 7, 11) == (2 * 32 * 7 + 68 * (2 * 3 + 2 * 5) + 64 + 11 + 15) // 16 * 16
    assert lib.bsa_attn_bwd_scratch_bytes(-1, 3, 5, 7, 11) == 0
    # room for dS, a buffer of its own: 8 KiB per block of the attention layout, 64 x 64 blocks only
    assert lib.bsa_attn_bwd_ds_bytes(7, 64) == 7 * 8192
    assert lib.bsa_attn_bwd_ds_bytes(-7, 64) == 0 and lib.bsa_attn_bwd_ds_bytes(7, 32) == 0
    # work orders built on the device: sizes, part counts, the table's length, the bound on a row's pairs
    assert lib.bsa_lut_block_order(0, -1, 4, 4, 16, 0, 0, 0, 0) == -1 and b"number of blocks" in lib.bsa_last_error()
    assert lib.bsa_lut_block_order(0, 4, 4, 4, 0, 0, 0, 0, 0) == -1 and b"tile size" in lib.bsa_last_error()
    assert lib.bsa_lut_block_order(0, 0, 4, 4, 16, 0, 0, 0, 0) == 0  # nothing to order
    assert lib.bsa_lut_row_work_table(0, 0, 8, 4, 4, 0, 10, 0, 0, 8, 0, 0, 0) == -1 and b"parts_log2" in lib.bsa_last_error()
    assert lib.bsa_lut_row_work_table(0, 0, 9, 3, 1, 0, 10, 0, 0, 8, 0, 0, 0) == -1 and b"are needed" in lib.bsa_last_error()
    assert lib.bsa_lut_row_work_table(0, 0, 9, 3, 1, 0, -1, 0, 0, 32, 0, 0, 0) == -1 and b"bound" in lib.bsa_last_error()
    assert lib.bsa_lut_row_work_table(0, 0, 0, 3, 1, 0, 10, 0, 0, 0, 0, 0, 0) == 0  # no rows
    # lists over pairs of rows: sizes, the 28 bits of a column, pointers
    assert lib.bsa_lut_pair_union(0, 1, -2, 4, 0, 0) == -1 and b"negative size" in lib.bsa_last_error()
    assert lib.bsa_lut_pair_union(0, 1, 2, 4, 0, 0) == -1 and b"NULL" in lib.bsa_last_error()
    assert lib.bsa_lut_pair_union(0, 0, 2, 4, 0, 0) == 0
    assert lib.bsa_lut_pair_entries(0, 0, 1, 2, 1 << 28, 0, 0) == -1 and b"too many columns" in lib.bsa_last_error()
    assert lib.bsa_lut_pair_entries(0, 0, 1, 2, 4, 0, 0) == -1 and b"NULL" in lib.bsa_last_error()
    assert lib.bsa_lut_pair_entries(0, 0, 1, 0, 4, 0, 0) == 0
    # records of the row kernel: parts_log2 in 0..3; without a table the rows are taken whole and in order
    assert lib.bsa_matmul_rows_records(0, 4, 4, 0, 0, 0, 4, 4, 0, 0, 0) == -1 and b"parts_log2" in lib.bsa_last_error()
    assert lib.bsa_matmul_rows_records(0, 8, 1, 0, 0, 0, 4, 4, 0, 0, 0) == -1 and b"work table" in lib.bsa_last_error()
    assert lib.bsa_matmul_rows_records(0, 8, 1, 0, 0, 0, 4, 129, 0, 0, 0) == -1 and b"at most 64" in lib.bsa_last_error()
    assert lib.bsa_matmul_rows_records(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0) == 0
    assert lib.bsa_matmul_rows(0, 0, 0, 0, 0, 0, 4, 1, 4, 1, 1, 32, _capi.BF16, 0) == -1 and b"sbs must be 64" in lib.bsa_last_error()
    # mask blocks that mask everything: 64 x 64 blocks only, no mask blocks is nothing to do
    assert lib.bsa_attn_mask_dead(0, 1, 32, 0, 0) == -1 and b"64 x 64" in lib.bsa_last_error()
    assert lib.bsa_attn_mask_dead(0, 1, 64, 0, 0) == -1 and b"NULL" in lib.bsa_last_error()
    assert lib.bsa_attn_mask_dead(0, 0, 64, 0, 0) == 0


def test_bad_arguments_of_the_line_kernel_are_rejected_on_the_host():
    """bsa_matmul_lines / bsa_matmul_lines_parts check their argument block before anything is launched."""
    import ctypes
    lib = _capi.load()
    a = _capi.LinesArgs()
    assert lib.bsa_matmul_lines(None, 0, 64, _capi.BF16, 0) == -1 and b"NULL argument block" in lib.bsa_last_error()
    a.n_batches, a.lines_per_batch, a.n_streamed, a.n_outputs = 1, 1, 513, 4
    assert lib.bsa_matmul_lines(ctypes.byref(a), 0, 64, _capi.BF16, 0) == -1
    assert b"at most 512 streamed blocks" in lib.bsa_last_error()
    a.n_streamed, a.n_outputs = 4, 600
    assert lib.bsa_matmul_lines(ctypes.byref(a), 0, 64, _capi.BF16, 0) == -1
    assert b"at most 512 output blocks" in lib.bsa_last_error()
    a.n_outputs = 4
    assert lib.bsa_matmul_lines(ctypes.byref(a), 0, 32, _capi.BF16, 0) == -1 and b"sbs must be 64" in lib.bsa_last_error()
    assert lib.bsa_matmul_lines(ctypes.byref(a), 0, 64, _capi.F32, 0) == -1 and b"fp16 or bf16" in lib.bsa_last_error()
    a.nnz_out = -1
    assert lib.bsa_matmul_lines(ctypes.byref(a), 0, 64, _capi.BF16, 0) == -1 and b"negative block count" in lib.bsa_last_error()
    a.nnz_out = 0
    assert lib.bsa_matmul_lines(ctypes.byref(a), 1, 64, _capi.BF16, 0) == 0  # no output block: nothing to do
    assert lib.bsa_matmul_lines_parts(ctypes.byref(a), 0, 0, 0) == -1 and b"NULL pointer" in lib.bsa_last_error()
    # the argument block mirrors the header: 7 pointers, 4 + 9 + 3 int64, one pointer
    assert ctypes.sizeof(_capi.LinesArgs) == 7 * 8 + 4 * 8 + 9 * 8 + 3 * 8 + 8
    assert _capi.LinesArgs.error.offset == 23 * 8 and _capi.LinesArgs.streamed_strides.offset == 11 * 8
