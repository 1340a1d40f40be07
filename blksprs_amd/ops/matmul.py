"""Block-sparse matrix multiplication of two compressed tensors.

Signature, validation order, error texts and the observable cache keys follow the
reference (blksprs/ops/matmul.py:17-67 wrapper, :256-279 cache, :130-145 backward).
The product itself walks per-output-block contraction lists built on the device
and is computed by ``bsa_matmul``.  The backward pass reads the saved operands
transposed inside the kernel instead of materialising transposed copies.
"""

import ctypes
import os
import warnings

import torch
from torch import Tensor

from .. import _capi
from ..utils.blksprs_tensor import BlksprsTensor
from ..utils.tools import (build_contraction_lists, cast_for_autocast, count_contraction_pairs, eager_only,
                           finalize_layout_cache, nonzero_from_packed, pack_layouts, prepare_layout_cache,
                           write_contraction_pairs)
from ..utils.validation import (ensure_contiguous, validate_contiguous, validate_device, validate_dimensions,
                                validate_dtype_float, validate_shape, validate_sparsity, validate_sparsity_block_size,
                                validate_sparsity_layout, validation_enabled)


def _launch(x: Tensor, y: Tensor, pair_offsets: Tensor, pairs: Tensor, order: Tensor | None, n_out: int, sbs: int,
            trans_x: bool, trans_y: bool) -> Tensor:
    out = torch.empty((n_out, sbs, sbs), dtype=x.dtype, device=x.device)
    if n_out:
        with _capi.on_device(x.device):
            # x and y may be empty (no block at all): the library never reads an operand of zero blocks
            _capi.call("bsa_matmul", x.data_ptr(), y.data_ptr(), out.data_ptr(), pair_offsets.data_ptr(),
                       _capi.ptr(pairs), _capi.ptr(order), n_out, x.size(0), y.size(0), sbs,
                       _capi.DTYPE_CODES[x.dtype], int(trans_x), int(trans_y), _capi.stream(x.device))
    return out


def _launch_rows(x: Tensor, y: Tensor, plan: "_Plan", sbs: int) -> Tensor:
    """Forward product by output block row (fp16 / bf16, sbs 64): x row panels stay in LDS."""
    n_out = plan.n_out
    out = torch.empty((n_out, sbs, sbs), dtype=x.dtype, device=x.device)
    if n_out:
        with _capi.on_device(x.device):
            _capi.call("bsa_matmul_rows", _capi.ptr(x), _capi.ptr(y), out.data_ptr(),
                       plan.pair_offsets.data_ptr(), _capi.ptr(plan.pairs),
                       _capi.ptr(plan.row_records), plan.row_records.size(0), plan.row_items, n_out,
                       x.size(0), y.size(0), sbs, _capi.DTYPE_CODES[x.dtype], _capi.stream(x.device))
    return out


_MAX_LINE_BLOCKS = 512  # blocks per line that the line kernel's lists in LDS hold


def _lines_args(plan: "_Plan", shapes, which: str, streamed: Tensor | None, private: Tensor | None,
                out: Tensor | None, part_table: Tensor | None) -> _capi.LinesArgs:
    """Argument block of the line kernel for dX = dO Y^T (``which == "x"``: lines are the block rows of x) or
    dY = X^T dO (``"y"``: the block columns of y).  The streamed operand is dO in both."""
    (B, R, K), (_, _, C) = shapes
    a = _capi.LinesArgs()
    a.n_batches = B
    a.pidx_streamed = _capi.ptr(plan.packed_o)
    a.nnz_streamed = plan.n_out
    if which == "x":
        a.lines_per_batch, a.n_streamed, a.n_outputs = R, C, K
        a.streamed_strides[:] = (R * C, C, 1)
        a.pidx_out, a.out_strides[:] = _capi.ptr(plan.packed_x), (R * K, K, 1)
        a.pidx_private, a.private_strides[:] = _capi.ptr(plan.packed_y), (K * C, C, 1)
        a.nnz_out, a.nnz_private = plan.n_x, plan.n_y
    else:
        a.lines_per_batch, a.n_streamed, a.n_outputs = C, R, K
        a.streamed_strides[:] = (R * C, 1, C)
        a.pidx_out, a.out_strides[:] = _capi.ptr(plan.packed_y), (K * C, 1, C)
        a.pidx_private, a.private_strides[:] = _capi.ptr(plan.packed_x), (R * K, 1, K)
        a.nnz_out, a.nnz_private = plan.n_y, plan.n_x
    a.streamed, a.priv, a.out = _capi.ptr(streamed), _capi.ptr(private), _capi.ptr(out)
    a.part_table = _capi.ptr(part_table)
    a.error = _capi.ptr(plan.lines_error)
    return a


def _lines_apply(plan: "_Plan", shapes, sbs: int, dtype: torch.dtype) -> bool:
    """Whether the two backward products run on the line kernel: 16-bit operands, 64 x 64 blocks, lines of dO and
    of the output of at most 512 blocks either way, fewer than 2^25 lines (an entry of the part table holds the line
    in 25 bits); everything else takes the tile kernel."""
    (B, R, K), (_, _, C) = shapes
    return (sbs == 64 and dtype in (torch.float16, torch.bfloat16) and max(R, C, K) <= _MAX_LINE_BLOCKS
            and B * max(R, C) < 2 ** 25)


def _lines_parts(plan: "_Plan", shapes) -> tuple[Tensor, Tensor]:
    """The part tables of the two backward products (``bsa_matmul_lines_parts``), built once per plan on the
    device; nothing is read back."""
    if plan.grad_lines is None:
        device = plan.packed_o.device
        plan.lines_error = torch.zeros(32, dtype=torch.int32, device=device)
        built = []
        for which in ("x", "y"):
            a = _lines_args(plan, shapes, which, None, None, None, None)
            n_lines = a.n_batches * a.lines_per_batch
            scratch = torch.empty(4 * n_lines + 2, dtype=torch.int32, device=device)
            table = torch.empty(1 + a.nnz_out // 16 + n_lines, dtype=torch.int32, device=device)
            with _capi.on_device(device):
                _capi.call("bsa_matmul_lines_parts", ctypes.byref(a), scratch.data_ptr(), table.data_ptr(),
                           _capi.stream(device))
            built.append(table)
        plan.grad_lines = tuple(built)
    return plan.grad_lines


def _launch_lines(plan: "_Plan", shapes, which: str, streamed: Tensor, private: Tensor, n_out: int, sbs: int) -> Tensor:
    out = torch.empty((n_out, sbs, sbs), dtype=streamed.dtype, device=streamed.device)
    if n_out:
        table = _lines_parts(plan, shapes)[0 if which == "x" else 1]
        a = _lines_args(plan, shapes, which, streamed, private, out, table)
        with _capi.on_device(streamed.device):
            _capi.call("bsa_matmul_lines", ctypes.byref(a), int(which == "y"), sbs, _capi.DTYPE_CODES[streamed.dtype],
                       _capi.stream(streamed.device))
    return out


_SUPER_TILE = 16


def _block_order(layout_indices: Tensor, n_rows: int, n_cols: int) -> Tensor:
    """Work order of the output blocks of a layout with ``n_rows`` x ``n_cols`` blocks per batch entry: 16 x 16
    super-tiles of the block grid, columns of super-tiles fastest, so that the blocks in flight on one L2 share
    x row panels and y column panels (``bsa_lut_block_order``: built on the device, nothing is read back)."""
    layout_indices = layout_indices.contiguous()  # torch.nonzero hands out column-major results
    n = layout_indices.size(0)
    order = torch.empty(n, dtype=torch.int32, device=layout_indices.device)
    if n:
        ws_bytes = _capi.load().bsa_lut_order_workspace_bytes(n)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=layout_indices.device)
        with _capi.on_device(layout_indices.device):
            _capi.call("bsa_lut_block_order", layout_indices.data_ptr(), n, n_rows, n_cols, _SUPER_TILE,
                       order.data_ptr(), workspace.data_ptr(), ws_bytes, _capi.stream(layout_indices.device))
    return order


_N_XCD = 8


_L2_BYTES = 4 << 20  # one XCD's L2


_MAX_PART_BLOCKS = 64  # a workgroup of the row kernel takes at most this many output blocks (one mask bit each)


def _measurement_knob(name: str, default: int, lowest: int, highest: int) -> int:
    """An integer from the environment for measurements of the row kernel's work order, clamped to its legal
    range; a value that is not a number is ignored with a warning (a value left over in the environment must not
    turn every product into an error)."""
    raw = os.environ.get(name)
    if raw is None:
        return default
    try:
        value = int(raw)
    except ValueError:
        warnings.warn(f"{name}={raw!r} is not an integer: ignored")
        return default
    return min(max(value, lowest), highest)


def _row_parts_log2(n_rows: int, rows_per_batch: int, n_cols: int, n_blocks_y: int, n_blocks_o: int,
                    block_bytes: int) -> int | None:
    """Into how many runs (as log2) the row kernel cuts the output blocks of a row; ``None`` when a row does not
    fit the kernel's eight parts.

    The rows in flight on one XCD belong to one batch entry and walk its y blocks column by column, roughly in
    step, so the y blocks in flight are a band of columns.  When an entry's y blocks are several times an
    XCD's L2, two column halves of the entry, one after the other, halve the band; the x row is then loaded
    twice, and with four parts that costs more than it saves.  Rows too short to feed eight waves twice stay
    whole.  A part holds at most 64 blocks.
    """
    batches = max(n_rows // max(rows_per_batch, 1), 1)
    y_bytes_per_entry = n_blocks_y * block_bytes // batches
    blocks_per_row = n_blocks_o // max(n_rows, 1)
    parts_log2 = 1 if y_bytes_per_entry > 4 * _L2_BYTES and blocks_per_row >= 32 else 0
    parts_log2 = _measurement_knob("BLKSPRS_AMD_ROW_PARTS_LOG2", parts_log2, 0, 3)
    while parts_log2 <= 3 and -(-n_cols // (1 << parts_log2)) > _MAX_PART_BLOCKS:
        parts_log2 += 1
    return parts_log2 if parts_log2 <= 3 else None


def _row_records(work_table: Tensor, parts_log2: int, pair_offsets: Tensor, row_offsets_x: Tensor,
                 row_offsets_o: Tensor, n_rows: int, n_cols: int, n_blocks_x: int) -> Tensor:
    """One record per work table entry with what a workgroup of the row kernel needs to know about its part of
    a row (``bsa_matmul_rows_records``): int32 ``[n_items, 32]``."""
    records = torch.empty((work_table.numel(), _capi.ROWS_RECORD_INTS), dtype=torch.int32,
                          device=work_table.device)
    if work_table.numel():
        with _capi.on_device(work_table.device):
            _capi.call("bsa_matmul_rows_records", _capi.ptr(work_table), work_table.numel(), parts_log2,
                       pair_offsets.data_ptr(), row_offsets_x.data_ptr(), row_offsets_o.data_ptr(), n_rows, n_cols,
                       n_blocks_x, _capi.ptr(records), _capi.stream(work_table.device))
    return records


_ROWS_DOWNWARD = 1 << 30  # BSA_ROWS_DOWNWARD
_CUS_PER_XCD = 32


def _row_work_table(pair_offsets: Tensor, row_offsets_o: Tensor, rows_per_batch: int, parts_log2: int,
                    pair_up: bool = False, max_work: int = 0, sweep: int = 0) -> Tensor:
    """Order in which the row kernel hands parts of output block rows to workgroups: int32 entries
    ``row << parts_log2 | part``, -1 for nothing (``bsa_lut_row_work_table``: built on the device, nothing is read
    back).

    Workgroup ``g`` runs on XCD ``g % 8``.  Every XCD gets one contiguous eighth of the rows (so the rows in
    flight on one L2 belong to the same batch entry and stream through the same y blocks), and walks it batch
    entry by batch entry, part by part, rows with the most (x, y) pairs first, so that the last workgroups of a
    launch are the short ones.  The k-th item of eighth c sits at position 8 k + c; eighths with a row less end
    in an empty entry.  With ``pair_up`` the rows of a batch entry alternate longest, shortest, second longest,
    second shortest, ...: a workgroup that takes two consecutive entries of its XCD's list then has about the
    same work as every other one, the workgroups of an XCD start and end their rows of one batch entry together
    (they stream through the same y blocks at the same time), and a launch ends without a tail of short rows.
    With ``sweep`` > 0 the items of one (XCD, batch entry, part) group alternate their direction every ``sweep``
    items: the first ``sweep`` walk their columns upward, the next ``sweep`` (which start as those end, on the
    same compute units) downward, and so on: a part that starts finds the y blocks its predecessors read last
    still in the L2.
    ``max_work`` is a bound on the pairs of one row that the caller knows without asking the device (inner
    blocks times output columns).
    """
    n_rows = row_offsets_o.numel() - 1
    parts = 1 << parts_log2
    device = row_offsets_o.device
    table = torch.empty((-(-n_rows // _N_XCD)) * parts * _N_XCD, dtype=torch.int32, device=device)
    if n_rows > 0:
        ws_bytes = _capi.load().bsa_lut_order_workspace_bytes(n_rows * parts)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=device)
        with _capi.on_device(device):
            _capi.call("bsa_lut_row_work_table", pair_offsets.data_ptr(), row_offsets_o.data_ptr(), n_rows,
                       rows_per_batch, parts_log2, int(pair_up), int(max_work), int(sweep), table.data_ptr(),
                       table.numel(), workspace.data_ptr(), ws_bytes, _capi.stream(device))
    return table


class _Plan:
    """The lookup tables of one (x layout, y layout, output layout) triple as one object.  A forward pass hands
    this object, not the caller's cache dict, to its backward pass: the dict may be emptied and filled for other
    layouts between the two (``prepare_layout_cache`` clears it in place), the object keeps what it was built
    with.  Nothing writes to its tensors after they are built."""

    __slots__ = ("pair_offsets", "pairs", "block_order", "n_out", "n_x", "n_y", "row_records", "row_items",
                 "packed_x", "packed_y", "packed_o", "grad_lists", "grad_lines", "lines_error")

    def __init__(self, cache: dict):
        self.pair_offsets, self.pairs = cache["contraction_offsets"], cache["contraction_pairs"]
        self.block_order, self.row_records = cache["block_order"], cache["row_records"]
        self.row_items = cache["row_items_per_workgroup"]
        self.n_out, self.n_x, self.n_y = (cache["n_sparse_blocks"], cache["n_sparse_blocks_x"],
                                          cache["n_sparse_blocks_y"])
        self.packed_x, self.packed_y, self.packed_o = (cache["packed_indices_x"], cache["packed_indices_y"],
                                                       cache["packed_indices_o"])
        self.grad_lists = None  # contraction lists of the two backward products (tile kernel)
        self.grad_lines = self.lines_error = None  # part offsets of the two backward products (line kernel)


def _backward_lists(plan: _Plan, shape_x, shape_y):
    """Contraction lists of dX = dO Y^T and dY = X^T dO, built once per plan from the plan's own indices."""
    if plan.grad_lists is None:
        B, R, K = (int(s) for s in shape_x)
        C = int(shape_y[2])
        # operand layouts seen by the builder: dO (B,R,C) times Y^T (B,C,K) -> (B,R,K)
        pidx_yt = plan.packed_y.view(B, K, C).transpose(1, 2).contiguous().view(-1)
        # X^T (B,K,R) times dO (B,R,C) -> (B,K,C)
        pidx_xt = plan.packed_x.view(B, R, K).transpose(1, 2).contiguous().view(-1)
        # both products' pair counts come back in one read
        gx, gy = build_contraction_lists((plan.packed_o, pidx_yt, plan.packed_x, B, R, C, K, plan.n_x),
                                         (pidx_xt, plan.packed_o, plan.packed_y, B, K, R, C, plan.n_y))
        plan.grad_lists = (gx.pair_offsets, gx.pairs, gy.pair_offsets, gy.pairs)
    return plan.grad_lists


def _publish_backward_lists(layout_cache: dict, plan: _Plan) -> None:
    """Shows the plan's backward tables under the cache's own keys, while the cache still belongs to the plan."""
    if layout_cache.get("plan") is not plan:
        return
    if plan.grad_lists is not None and "grad_x_pair_offsets" not in layout_cache:
        (layout_cache["grad_x_pair_offsets"], layout_cache["grad_x_pairs"], layout_cache["grad_y_pair_offsets"],
         layout_cache["grad_y_pairs"]) = plan.grad_lists
        finalize_layout_cache(layout_cache)
    if plan.grad_lines is not None and "grad_x_part_table" not in layout_cache:
        layout_cache["grad_x_part_table"], layout_cache["grad_y_part_table"] = plan.grad_lines
        layout_cache["grad_lines_error"] = plan.lines_error
        finalize_layout_cache(layout_cache)


def _forward(x: Tensor, y: Tensor, plan: _Plan, sparsity_block_size: int) -> Tensor:
    if (sparsity_block_size == 64 and x.dtype in (torch.float16, torch.bfloat16)
            and plan.row_records is not None):
        return _launch_rows(x, y, plan, sparsity_block_size)
    return _launch(x, y, plan.pair_offsets, plan.pairs, plan.block_order, plan.n_out, sparsity_block_size,
                   False, False)


class _Matmul(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, y, layout_cache, shape_x, shape_y, sparsity_block_size):
        plan = layout_cache["plan"]
        ctx.save_for_backward(x, y)
        ctx.plan = plan
        ctx.layout_cache = layout_cache  # only to publish the backward lists; never read for the computation
        ctx.shapes = (shape_x, shape_y)
        ctx.sparsity_block_size = sparsity_block_size
        return _forward(x, y, plan, sparsity_block_size)

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        x, y = ctx.saved_tensors
        sbs = ctx.sparsity_block_size
        plan = ctx.plan
        grad_x = grad_y = None
        if _lines_apply(plan, ctx.shapes, sbs, x.dtype):
            # by lines of dO (row i for dX, column j for dY), each streamed through LDS once
            _lines_parts(plan, ctx.shapes)
            _publish_backward_lists(ctx.layout_cache, plan)
            if ctx.needs_input_grad[0]:
                grad_x = _launch_lines(plan, ctx.shapes, "x", grad_output, y, x.size(0), sbs)
            if ctx.needs_input_grad[1]:
                grad_y = _launch_lines(plan, ctx.shapes, "y", grad_output, x, y.size(0), sbs)
            return grad_x, grad_y, None, None, None, None
        gx_off, gx_pairs, gy_off, gy_pairs = _backward_lists(plan, *ctx.shapes)
        _publish_backward_lists(ctx.layout_cache, plan)
        if ctx.needs_input_grad[0]:
            grad_x = _launch(grad_output, y, gx_off, gx_pairs, None, x.size(0), sbs, False, True)
        if ctx.needs_input_grad[1]:
            grad_y = _launch(x, grad_output, gy_off, gy_pairs, None, y.size(0), sbs, True, False)
        return grad_x, grad_y, None, None, None, None


def matmul_build_layout_cache(layout_cache: dict | None, sparsity_layout_x: Tensor, sparsity_layout_y: Tensor,
                              sparsity_layout_output: Tensor) -> dict:
    """Fills the cache of one (x layout, y layout, output layout) triple.

    Keys shared with the reference: ``packed_indices_x``, ``packed_indices_y`` (int64, flat),
    ``layout_indices_o`` (int64 ``[n, 3]``), ``n_sparse_blocks``.  Additional keys hold the
    contraction lists the kernel walks (``contraction_offsets`` int32 ``[n + 1]``,
    ``contraction_pairs`` int32 ``[pairs, 2]``) and the counts they were sized with.
    """
    layout_cache = prepare_layout_cache(layout_cache, "matmul", sparsity_layout_x, sparsity_layout_y,
                                        sparsity_layout_output)
    if "contraction_pairs" not in layout_cache:
        B, R, K = (int(s) for s in sparsity_layout_x.shape)
        C = int(sparsity_layout_y.size(2))
        # the three scans and the count of the product's block pairs are launched one after the other, and
        # their results (block counts, longest rows, number of pairs) come back in ONE read
        counted = []
        (info_x, info_y, info_o), (n_pairs, _) = pack_layouts(
            (sparsity_layout_x, K), (sparsity_layout_y, 0), (sparsity_layout_output, C),
            then=lambda packed: (counted.append(count_contraction_pairs(*packed, B, R, K, C)), counted[0].stats_dev)[1])
        lists = write_contraction_pairs(counted[0], int(n_pairs), info_o.count)
        layout_cache["packed_indices_x"] = info_x.packed
        layout_cache["packed_indices_y"] = info_y.packed
        layout_cache["packed_indices_o"] = info_o.packed
        layout_cache["layout_indices_o"] = nonzero_from_packed(info_o.packed, sparsity_layout_output.shape,
                                                               info_o.count)
        layout_cache["n_sparse_blocks"] = info_o.count
        layout_cache["n_sparse_blocks_x"] = info_x.count
        layout_cache["n_sparse_blocks_y"] = info_y.count
        layout_cache["contraction_offsets"] = lists.pair_offsets
        layout_cache["contraction_pairs"] = lists.pairs
        layout_cache["block_order"] = _block_order(layout_cache["layout_indices_o"], R, C)
        layout_cache["row_offsets_x"] = info_x.row_offsets
        layout_cache["row_offsets_o"] = info_o.row_offsets
        layout_cache["row_records"] = None
        layout_cache["row_items_per_workgroup"] = 1
        if info_x.row_offsets is not None and info_o.row_offsets is not None:
            parts_log2 = _row_parts_log2(B * R, R, C, info_y.count, info_o.count, 64 * 64 * 2)
            if parts_log2 is not None:
                # One row per workgroup.  Two per workgroup, a long one and a short one (equal work for every
                # workgroup, no tail of short rows), measured no faster on configuration 2: compute units differ
                # in speed by +-12 % on equal work, which the hardware's hand-out of many small items evens out
                # and a static split does not.  Kept switchable for measurements.
                pair_up = (B * R << parts_log2) >= 1024 and _measurement_knob("BLKSPRS_AMD_ROW_PAIRS", 0, 0, 1) == 1
                sweep = _measurement_knob("BLKSPRS_AMD_ROW_SWEEP", _CUS_PER_XCD, 0, 1 << 20)  # 0: every part upward
                table = _row_work_table(lists.pair_offsets, info_o.row_offsets, R, parts_log2, pair_up,
                                        max_work=K * C, sweep=0 if pair_up else sweep)
                layout_cache["row_parts_log2"], layout_cache["row_work_table"] = parts_log2, table
                layout_cache["row_items_per_workgroup"] = 2 if pair_up else 1
                layout_cache["row_records"] = _row_records(table, parts_log2, lists.pair_offsets,
                                                           info_x.row_offsets, info_o.row_offsets, B * R, C,
                                                           info_x.count)
        layout_cache["plan"] = _Plan(layout_cache)

    validate_contiguous(sparsity_layout_x, layout_cache["packed_indices_x"],
                        sparsity_layout_y, layout_cache["packed_indices_y"],
                        sparsity_layout_output, layout_cache["layout_indices_o"])
    return finalize_layout_cache(layout_cache)


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def matmul(x: BlksprsTensor, sparsity_layout_x: Tensor,
           y: BlksprsTensor, sparsity_layout_y: Tensor,
           sparsity_layout_output: Tensor,
           sparsity_block_size: int, layout_cache: dict | None = None) -> BlksprsTensor:
    """Multiplies two compressed block-sparse tensors.

    Only blocks marked active by ``sparsity_layout_output`` are calculated.

    Args:
        x (BlksprsTensor): The compressed left operand.
        sparsity_layout_x (Tensor): The sparsity layout of ``x``.
        y (BlksprsTensor): The compressed right operand.
        sparsity_layout_y (Tensor): The sparsity layout of ``y``.
        sparsity_layout_output (Tensor): The sparsity layout of the output tensor.
        sparsity_block_size (int): The size of the sparsity blocks.
        layout_cache (dict, optional): Reusable layout metadata cache (default ``None``).

    Returns:
        BlksprsTensor: The matrix product in compressed form.

    """
    x, y = ensure_contiguous(x, y)
    x, y = cast_for_autocast(x, y)

    if validation_enabled():  # every check below is a no-op otherwise
        validate_dimensions(x, y)
        validate_contiguous(x, y, sparsity_layout_output)
        validate_dtype_float(x, y)
        validate_device(x, y, sparsity_layout_output)
        validate_sparsity(sparsity_block_size, (x, sparsity_layout_x), (y, sparsity_layout_y))
        validate_sparsity_layout(sparsity_layout_output)
    if sparsity_layout_x.size(0) != sparsity_layout_y.size(0):
        raise ValueError("Batch dimensions of tensors must match")
    if sparsity_layout_x.size(-1) != sparsity_layout_y.size(-2):
        raise ValueError("Inner dimensions of tensors must match")
    if validation_enabled():
        validate_shape(
            sparsity_layout_output,
            (sparsity_layout_x.size(0), sparsity_layout_x.size(1), sparsity_layout_y.size(2)),
            "Output sparsity layout",
        )
        validate_sparsity_block_size(sparsity_block_size, x, y)

    layout_cache = matmul_build_layout_cache(layout_cache, sparsity_layout_x, sparsity_layout_y,
                                             sparsity_layout_output)

    if not (torch.is_grad_enabled() and (x.requires_grad or y.requires_grad)):
        # nothing to differentiate: the launch itself, without the autograd machinery around it
        return BlksprsTensor.wrap(_forward(x, y, layout_cache["plan"], sparsity_block_size))
    shape_x, shape_y = tuple(sparsity_layout_x.shape), tuple(sparsity_layout_y.shape)
    plan = layout_cache["plan"]
    if plan.grad_lists is None and not _lines_apply(plan, (shape_x, shape_y), sparsity_block_size, x.dtype):
        # the lists of the two backward products are built with the first forward pass that will need them, so
        # that no backward pass waits for the device (the line kernel needs no lists, and its part offsets are
        # built without a read by the host)
        _backward_lists(plan, shape_x, shape_y)
        _publish_backward_lists(layout_cache, plan)
    return BlksprsTensor.wrap(_Matmul.apply(x, y, layout_cache, shape_x, shape_y, sparsity_block_size))
