"""Row-wise sum, maximum and add over the active blocks of a compressed tensor.

Public behaviour follows blksprs/ops/misc/row_wise.py: signatures and validation (:35-100, :235-280,
:420-466), the output layout ``any(layout, -1, keepdim=True)`` (:74-76), square output blocks whose first
column holds the result or ``(rows, sbs, 1)`` slices with ``flag_slice_only`` (:43-47), fp32 accumulation with
one rounding to the input dtype (:108-114, :146), NaN and -inf behaviour of the maximum (:300-310, :349-350),
and the early return for empty inputs (:84-93).  None of the operations records a gradient.

The reference takes no layout cache here and rebuilds its lookup tables on every call (:71-78); this module
keeps the tables of the last few layouts it saw, filed under the identity and in-place version of the layout
tensor, so a loop over one layout pays for them once.
"""

import threading
from collections import OrderedDict

import torch
from torch import Tensor

from ... import _capi
from ...utils.blksprs_tensor import BlksprsTensor
from ...utils.tools import as_base_tensor, layout_cache_key, nonzero_from_packed, pack_layout
from ...utils.validation import (ensure_contiguous, validate_contiguous, validate_device, validate_dimensions,
                                 validate_dtype_float, validate_sparsity, validate_sparsity_block_size)

_SUM, _MAX = 0, 1


def _row_layout(sparsity_layout: Tensor) -> Tensor:
    """``(B, R, 1)`` layout of the block rows that hold at least one block."""
    return as_base_tensor(torch.any(as_base_tensor(sparsity_layout), dim=-1, keepdim=True))


class _Tables:
    """Lookup tables of one layout: its ``(B, R, 1)`` row layout, CSR offsets of the block rows, the reverse
    index of the row layout, the number of block rows that hold a block, and (on demand) the coordinates."""

    __slots__ = ("refs", "layout_rows", "row_offsets", "packed_rows", "n_rows_active", "packed", "count", "_coords")

    def __init__(self, sparsity_layout: Tensor, refs: tuple):
        self.refs = refs  # keeps the layout alive, so its identity cannot pass to another tensor
        self.layout_rows = _row_layout(sparsity_layout)
        info = pack_layout(sparsity_layout, row_len=int(sparsity_layout.size(-1)))
        rows = pack_layout(self.layout_rows)
        self.row_offsets, self.packed, self.count = info.row_offsets, info.packed, info.count
        self.packed_rows, self.n_rows_active = rows.packed, rows.count
        self._coords = None

    def coords(self, shape) -> Tensor:
        if self._coords is None:
            self._coords = nonzero_from_packed(self.packed, shape, self.count)
        return self._coords


_MEMO: "OrderedDict[tuple, _Tables]" = OrderedDict()
_MEMO_SIZE = 8
_MEMO_LOCK = threading.Lock()


def _tables(sparsity_layout: Tensor) -> _Tables:
    key, refs = layout_cache_key("row_wise", sparsity_layout)
    with _MEMO_LOCK:
        hit = _MEMO.get(key)
        if hit is not None:
            _MEMO.move_to_end(key)
            return hit
    tables = _Tables(sparsity_layout, refs)
    with _MEMO_LOCK:
        _MEMO[key] = tables
        while len(_MEMO) > _MEMO_SIZE:
            _MEMO.popitem(last=False)
    return tables


def _reduce(x: Tensor, sparsity_layout: Tensor, sparsity_block_size: int, flag_slice_only: bool,
            op: int) -> tuple[BlksprsTensor | Tensor, Tensor]:
    x = ensure_contiguous(x)

    validate_dimensions(x)
    validate_contiguous(x)
    validate_dtype_float(x)
    validate_device(x)
    validate_sparsity(sparsity_block_size, (x, sparsity_layout))
    validate_sparsity_block_size(sparsity_block_size, x)

    columns = 1 if flag_slice_only else sparsity_block_size
    wrap = as_base_tensor if flag_slice_only else BlksprsTensor.wrap

    if x.size(0) == 0:
        empty = torch.empty((0, sparsity_block_size, columns), dtype=x.dtype, device=x.device)
        return wrap(empty), _row_layout(sparsity_layout)

    tables = _tables(sparsity_layout)
    n_rows = int(sparsity_layout.size(0)) * int(sparsity_layout.size(1))
    with torch.no_grad():
        out = torch.empty((tables.n_rows_active, sparsity_block_size, columns), dtype=x.dtype, device=x.device)
        with _capi.on_device(x.device):
            _capi.call("bsa_row_reduce", x.data_ptr(), tables.row_offsets.data_ptr(), tables.packed_rows.data_ptr(),
                       _capi.ptr(out), n_rows, tables.n_rows_active, x.size(0), sparsity_block_size,
                       _capi.DTYPE_CODES[x.dtype], op, int(flag_slice_only), _capi.stream(x.device))
    # every call hands out a layout of its own, as the reference does
    return wrap(out), tables.layout_rows.clone()


def row_wise_sum(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                 flag_slice_only: bool = False) -> tuple[BlksprsTensor | Tensor, Tensor]:
    """Sum of every element row over the active blocks of its block row.

    Args:
        x (BlksprsTensor): The compressed input tensor (fp16, bf16 or fp32).
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        flag_slice_only (bool, optional): Return ``(rows, sbs, 1)`` slices (a plain tensor, accepted by
            :func:`row_wise_add` and :func:`row_wise_sub`) instead of square blocks (default ``False``).

    Returns:
        tuple[BlksprsTensor | Tensor, Tensor]: The row sums (first column of each block; the other columns are
            zero) and their ``(B, R, 1)`` layout with one block per block row that holds a block.
    """
    return _reduce(x, sparsity_layout, sparsity_block_size, flag_slice_only, _SUM)


def row_wise_max(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                 flag_slice_only: bool = False) -> tuple[BlksprsTensor | Tensor, Tensor]:
    """Maximum of every element row over the active blocks of its block row.

    A row that holds a NaN gives NaN; a row of ``-inf`` gives ``-inf``.

    Args:
        x (BlksprsTensor): The compressed input tensor (fp16, bf16 or fp32).
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        flag_slice_only (bool, optional): Return ``(rows, sbs, 1)`` slices (a plain tensor) instead of square
            blocks (default ``False``).

    Returns:
        tuple[BlksprsTensor | Tensor, Tensor]: The row maxima (first column of each block; the other columns are
            ``-inf``) and their ``(B, R, 1)`` layout.
    """
    return _reduce(x, sparsity_layout, sparsity_block_size, flag_slice_only, _MAX)


def row_wise_add(x: BlksprsTensor, sparsity_layout_x: Tensor, y: Tensor,
                 sparsity_block_size: int) -> BlksprsTensor:
    """Adds one value per element row to every element of that row of ``x``.

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout_x (Tensor): The sparsity layout of ``x``.
        y (Tensor): One block per block row of ``x`` that holds a block, either ``(rows, sbs, 1)`` slices or
            square blocks whose first column is used; same dtype as ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.

    Returns:
        BlksprsTensor: ``x`` with the row values added, in compressed form.
    """
    x, y = ensure_contiguous(x, y)

    validate_dimensions(x, y)
    validate_contiguous(x, y)
    validate_dtype_float(x, y)
    validate_device(x, y)
    validate_sparsity(sparsity_block_size, (x, sparsity_layout_x))
    validate_sparsity_block_size(sparsity_block_size, x)

    if sparsity_layout_x.numel():
        tables = _tables(sparsity_layout_x)
        n_rows_active = tables.n_rows_active
    else:
        tables, n_rows_active = None, 0
    if y.size(0) != n_rows_active:
        raise ValueError("Row-wise tensor does not conform to input sparsity layout")
    if y.size(-2) != sparsity_block_size or y.size(-1) not in (1, sparsity_block_size):
        raise ValueError(
            "Row-wise tensor blocks must have sparsity block size rows and either 1 or sparsity block size columns")

    with torch.no_grad():
        out = torch.empty_like(as_base_tensor(x))
        if x.size(0):
            coords = tables.coords(sparsity_layout_x.shape)
            with _capi.on_device(x.device):
                _capi.call("bsa_row_add", x.data_ptr(), coords.data_ptr(), tables.packed_rows.data_ptr(), _capi.ptr(y),
                           out.data_ptr(), x.size(0), y.size(0), int(sparsity_layout_x.size(0)),
                           int(sparsity_layout_x.size(1)), int(y.size(-1)), sparsity_block_size,
                           _capi.DTYPE_CODES[x.dtype], _capi.stream(x.device))
    return BlksprsTensor.wrap(out)


def row_wise_sub(x: BlksprsTensor, sparsity_layout_x: Tensor, y: Tensor,
                 sparsity_block_size: int) -> BlksprsTensor:
    """Subtracts one value per element row from every element of that row of ``x`` (blksprs/ops/misc/row_wise.py:468-485)."""
    return row_wise_add(x, sparsity_layout_x, torch.neg(y), sparsity_block_size)
