"""Row-wise softmax over the active blocks of a compressed tensor (fp32).

Public behaviour follows the reference: ``softmax`` / ``softmax_fused`` /
``softmax_regular`` signatures and dispatch (blksprs/ops/softmax.py:24-50, :54-90,
:374-434), the 131072-element limit of the fused entry point (:19, :419-429), the
cache keys of both variants (:342-358, :641-670) and the early return for empty
inputs (:414-415).  Both variants run the same single-pass kernel, ``bsa_softmax_fwd``;
what differs is which reference-visible metadata they leave in the cache.
"""

import torch
from torch import Tensor

from .. import _capi
from ..utils.blksprs_tensor import BlksprsTensor
from ..utils.tools import (ceil_pow2, eager_only, finalize_layout_cache, nonzero_from_packed, pack_layout,
                           prepare_layout_cache, sorted_rows_from_offsets)
from ..utils.validation import (ensure_contiguous, validate_contiguous, validate_device, validate_dimensions,
                                validate_dtype_float_32, validate_sparsity, validate_sparsity_block_size)

_FUSED_SOFTMAX_MAX_ROW_ELEMENTS = 131_072


class _Softmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, row_offsets, n_rows, sparsity_block_size):
        out = torch.empty_like(x)
        with _capi.on_device(x.device):
            _capi.call("bsa_softmax_fwd", x.data_ptr(), out.data_ptr(), row_offsets.data_ptr(), n_rows, x.size(0),
                       sparsity_block_size, _capi.stream(x.device))
        ctx.save_for_backward(out, row_offsets)
        ctx.n_rows = n_rows
        ctx.sparsity_block_size = sparsity_block_size
        return out

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        out, row_offsets = ctx.saved_tensors
        grad_x = torch.empty_like(out)
        with _capi.on_device(out.device):
            _capi.call("bsa_softmax_bwd", grad_output.data_ptr(), out.data_ptr(), grad_x.data_ptr(),
                       row_offsets.data_ptr(), ctx.n_rows, out.size(0), ctx.sparsity_block_size,
                       _capi.stream(out.device))
        return grad_x, None, None, None


def _scan_rows(layout_cache: dict, sparsity_layout: Tensor) -> None:
    """One device pass: CSR row offsets, reverse index, block count, longest row."""
    if "row_offsets" not in layout_cache:
        info = pack_layout(sparsity_layout, row_len=int(sparsity_layout.size(-1)))
        layout_cache["row_offsets"] = info.row_offsets
        layout_cache["packed_indices"] = info.packed
        layout_cache["n_sparse_blocks"] = info.count
        layout_cache["max_blocks_row"] = info.max_per_row


def softmax_fused_build_layout_cache(layout_cache: dict | None, sparsity_layout: Tensor) -> dict:
    """Metadata of the fused variant: ``packed_indices_sorted`` and ``max_blocks_line`` (a power of two >= 2)."""
    layout_cache = prepare_layout_cache(layout_cache, "softmax", sparsity_layout)
    _scan_rows(layout_cache, sparsity_layout)
    if "packed_indices_sorted" not in layout_cache:
        n_rows = int(sparsity_layout.size(0) * sparsity_layout.size(1))
        layout_cache["packed_indices_sorted"] = sorted_rows_from_offsets(
            layout_cache["row_offsets"], n_rows, int(sparsity_layout.size(2)))
    if "max_blocks_line" not in layout_cache:
        layout_cache["max_blocks_line"] = ceil_pow2(int(max(layout_cache["max_blocks_row"], 2)))
    validate_contiguous(sparsity_layout, layout_cache["packed_indices_sorted"])
    return finalize_layout_cache(layout_cache)


def softmax_build_layout_cache(layout_cache: dict | None, sparsity_layout: Tensor) -> dict:
    """Metadata of the regular variant: ``layout_indices`` and ``packed_indices_rws`` (reverse index of the
    per-row "any block active" column)."""
    layout_cache = prepare_layout_cache(layout_cache, "softmax", sparsity_layout)
    _scan_rows(layout_cache, sparsity_layout)
    if "layout_indices" not in layout_cache:
        layout_cache["layout_indices"] = nonzero_from_packed(layout_cache["packed_indices"], sparsity_layout.shape,
                                                             layout_cache["n_sparse_blocks"])
    if "packed_indices_rws" not in layout_cache:
        offsets = layout_cache["row_offsets"]
        rows_active = (offsets[1:] != offsets[:-1])
        layout_cache["packed_indices_rws"] = pack_layout(rows_active).packed
    validate_contiguous(sparsity_layout, layout_cache["layout_indices"], layout_cache["packed_indices_rws"])
    return finalize_layout_cache(layout_cache)


def _validate(x: Tensor, sparsity_layout: Tensor, sparsity_block_size: int) -> Tensor:
    x = ensure_contiguous(x)
    validate_dimensions(x)
    validate_contiguous(x)
    validate_dtype_float_32(x)
    validate_device(x)
    validate_sparsity(sparsity_block_size, (x, sparsity_layout))
    validate_sparsity_block_size(sparsity_block_size, x)
    return x


def _run(x: Tensor, sparsity_layout: Tensor, sparsity_block_size: int, layout_cache: dict) -> BlksprsTensor:
    n_rows = int(sparsity_layout.size(0) * sparsity_layout.size(1))
    return BlksprsTensor.wrap(_Softmax.apply(x, layout_cache["row_offsets"], n_rows, sparsity_block_size))


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def softmax(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
            flag_fused: bool = True, layout_cache: dict | None = None) -> BlksprsTensor:
    """Computes a row-wise block-sparse softmax.

    Inactive blocks do not participate (they are equivalent to ``-inf``); rows without an active block are
    left out.  ``flag_fused`` selects which metadata set is kept in ``layout_cache``; rows whose
    power-of-two-padded length exceeds 131,072 elements always use the regular metadata.

    Args:
        x (BlksprsTensor): The compressed input tensor (float32).
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        flag_fused (bool, optional): Whether to prefer the fused variant (default ``True``).
        layout_cache (dict, optional): Reusable layout metadata cache (default ``None``).

    Returns:
        BlksprsTensor: The row-wise softmax in compressed form.

    """
    if flag_fused:
        return _softmax_fused(x, sparsity_layout, sparsity_block_size, layout_cache, fallback_to_regular=True)
    return softmax_regular(x, sparsity_layout, sparsity_block_size, layout_cache)


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def softmax_regular(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                    layout_cache: dict | None = None) -> BlksprsTensor:
    """Row-wise softmax without a row-length limit (see :func:`softmax`)."""
    x = _validate(x, sparsity_layout, sparsity_block_size)
    if x.size(0) == 0:
        return BlksprsTensor.wrap(x)
    layout_cache = softmax_build_layout_cache(layout_cache, sparsity_layout)
    return _run(x, sparsity_layout, sparsity_block_size, layout_cache)


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def softmax_fused(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                  layout_cache: dict | None = None) -> BlksprsTensor:
    """Row-wise softmax restricted to rows of at most 131,072 power-of-two-padded elements.

    Raises:
        ValueError: If the padded row exceeds that limit; :func:`softmax` falls back instead.

    """
    return _softmax_fused(x, sparsity_layout, sparsity_block_size, layout_cache, fallback_to_regular=False)


def _softmax_fused(x, sparsity_layout, sparsity_block_size, layout_cache, fallback_to_regular: bool):
    x = _validate(x, sparsity_layout, sparsity_block_size)
    if x.size(0) == 0:
        return BlksprsTensor.wrap(x)
    layout_cache = softmax_fused_build_layout_cache(layout_cache, sparsity_layout)
    padded_row_elements = layout_cache["max_blocks_line"] * sparsity_block_size
    if padded_row_elements > _FUSED_SOFTMAX_MAX_ROW_ELEMENTS:
        if fallback_to_regular:
            return softmax_regular(x, sparsity_layout, sparsity_block_size, layout_cache)
        raise ValueError(
            "Fused softmax supports power-of-two-padded rows of at most "
            f"{_FUSED_SOFTMAX_MAX_ROW_ELEMENTS} elements, but this layout "
            f"requires {padded_row_elements}. Use softmax() for automatic "
            "fallback or softmax(..., flag_fused=False) explicitly."
        )
    return _run(x, sparsity_layout, sparsity_block_size, layout_cache)
