"""PyTorch modules applied to compressed block-sparse tensors (blksprs/utils/processing.py).

``apply_torch_linear`` / ``apply_torch_linear_cached`` (:27-207) multiply the compressed input with the layer's
weight through ``bs.ops.matmul`` and add the bias; ``apply_function_applicable_row_wise`` and its two wrappers
(:210-296) run a callable over the packed rows.  Signatures, validation, returned layouts, gradient flow to the
input, the weight and the bias, and the keys of the linear cache follow the reference.

One thing is done differently.  The reference copies the transposed weight once per batch entry so that it
fits a ``(B, K, N)`` layout (:48-52).  The compressed form of a ``(B, R, C)`` layout is, block for block, that of
the ``(1, B * R, C)`` layout, so here the batch entries are stacked into one tall operand and multiplied with a
single ``(1, K, N)`` copy of the weight: same result and block order, no replicated weight, and the gradient of
the weight comes out of the one product already summed over the batch.  With a bias every output block is
active, consecutive blocks are consecutive column blocks, and the bias is added by plain broadcasting.
"""

from collections.abc import Callable

import torch
from torch import Tensor, nn

from .blksprs_tensor import BlksprsTensor
from .tools import CacheHolder, as_base_tensor, finalize_layout_cache, prepare_layout_cache
from .validation import (ensure_contiguous, validate_contiguous, validate_device, validate_dimensions,
                         validate_dtype_float, validate_dtype_supported, validate_shape, validate_sparsity,
                         validate_sparsity_block_size)


def _validate_linear_dtypes(x: Tensor, weight: Tensor, bias: Tensor | None) -> None:
    """Same dtype for input and parameters, unless autocast will unify them (blksprs/utils/processing.py:18-24)."""
    tensors = (x, weight) if bias is None else (x, weight, bias)
    if torch.is_autocast_enabled():
        for tensor in tensors:
            validate_dtype_float(tensor)
    else:
        validate_dtype_float(*tensors)


def _weight_layout(weight: Tensor, sparsity_block_size: int, device) -> Tensor:
    return torch.ones((1, weight.size(1) // sparsity_block_size, weight.size(0) // sparsity_block_size),
                      dtype=torch.bool, device=device)


def _output_layout(sparsity_layout: Tensor, layout_w_t: Tensor, with_bias: bool) -> Tensor:
    """All blocks with a bias (it fills every block, also without input features); otherwise the rows of the
    input that hold a block, over all output columns (blksprs/utils/processing.py:55-64)."""
    B, R, _ = sparsity_layout.shape
    n_out = layout_w_t.size(2)
    if with_bias:
        return torch.ones((B, R, n_out), dtype=torch.bool, device=sparsity_layout.device)
    from ..layouting.sparsity_layout import build_sparsity_layout_matmul_fast
    stacked = build_sparsity_layout_matmul_fast(_stack(sparsity_layout), layout_w_t)
    return stacked.reshape(B, R, n_out)


def _stack(layout: Tensor) -> Tensor:
    """``(B, R, C)`` -> ``(1, B * R, C)``: the same blocks in the same order."""
    layout = as_base_tensor(layout)
    return layout.reshape(1, layout.size(0) * layout.size(1), layout.size(2))


def _project(x: Tensor, stacked_layout: Tensor, w_t_bs: Tensor, layout_w_t: Tensor, stacked_layout_output: Tensor,
             bias_blocks: Tensor | None, sparsity_block_size: int, layout_cache: dict | None) -> BlksprsTensor:
    from ..ops.matmul import matmul
    out = matmul(x, stacked_layout, BlksprsTensor.wrap(w_t_bs.to(x.dtype)), layout_w_t,
                 stacked_layout_output, sparsity_block_size, layout_cache=layout_cache)
    n_out = layout_w_t.size(2)
    if bias_blocks is not None and n_out:
        s = sparsity_block_size
        rows = out.size(0) // n_out
        out = (as_base_tensor(out).reshape(rows, n_out, s, s) + bias_blocks.to(out.dtype)).reshape(rows * n_out, s, s)
    return BlksprsTensor.wrap(out)


def _bias_blocks(bias: Tensor, sparsity_block_size: int) -> Tensor:
    """``(1, N / sbs, 1, sbs)``: the slice of the bias every row of column block ``n`` receives."""
    validate_sparsity_block_size(sparsity_block_size, bias.reshape(1, 1, -1).expand(1, sparsity_block_size, -1))
    return bias.reshape(1, -1, 1, sparsity_block_size)


def _compress_weight(weight: Tensor, layout_w_t: Tensor, sparsity_block_size: int) -> Tensor:
    from ..ops.conversion import to_sparse
    return to_sparse(weight.transpose(-1, -2).unsqueeze(0), layout_w_t, sparsity_block_size)


@torch.amp.custom_fwd(device_type="cuda")
def apply_torch_linear(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                       linear: nn.Linear, bias: nn.Parameter | None = None) -> tuple[BlksprsTensor, Tensor]:
    """Applies a PyTorch linear layer to a block-sparse tensor.

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        linear (nn.Linear): The linear layer to apply.
        bias (nn.Parameter, optional): An explicit bias overriding ``linear.bias`` (default ``None``).

    Returns:
        tuple[BlksprsTensor, Tensor]: The projected tensor in compressed form and its sparsity layout.
    """
    w = linear.weight
    b = bias if bias is not None else linear.bias
    _validate_linear_dtypes(x, w, b)
    validate_sparsity_block_size(sparsity_block_size, w)

    layout_w_t = _weight_layout(w, sparsity_block_size, x.device)
    layout_output = _output_layout(sparsity_layout, layout_w_t, b is not None)
    w_t_bs = _compress_weight(w, layout_w_t, sparsity_block_size)
    bias_blocks = _bias_blocks(b, sparsity_block_size) if b is not None else None
    out = _project(x, _stack(sparsity_layout), w_t_bs, layout_w_t, _stack(layout_output), bias_blocks,
                   sparsity_block_size, None)
    return out, layout_output


@torch.amp.custom_fwd(device_type="cuda")
def apply_torch_linear_cached(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                              linear: nn.Linear, bias: nn.Parameter | None = None,
                              layout_cache: dict | None = None) -> tuple[BlksprsTensor, Tensor]:
    """Applies a PyTorch linear layer while keeping its compressed parameters and lookup tables in a cache.

    The cache is rebuilt when the input layout, the block size, the device or dtype of ``x``, the gradient mode,
    or the identity, version or ``requires_grad`` of a parameter changes (blksprs/utils/processing.py:110-120).
    Keys: ``sparsity_layout_w_t``, ``w_t_bs``, ``sparsity_layout_output``, with a bias also ``bias_slice_bs``,
    and ``stacked_layouts`` / ``matmul_layout_cache`` for the product.

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        linear (nn.Linear): The linear layer to apply.
        bias (nn.Parameter, optional): An explicit bias overriding ``linear.bias`` (default ``None``).
        layout_cache (dict, optional): Reusable layout and parameter cache (default ``None``).

    Returns:
        tuple[BlksprsTensor, Tensor]: The projected tensor in compressed form and its sparsity layout.
    """
    w = linear.weight
    b = bias if bias is not None else linear.bias
    _validate_linear_dtypes(x, w, b)
    validate_sparsity_block_size(sparsity_block_size, w)

    layout_cache = prepare_layout_cache(layout_cache, "apply_torch_linear", sparsity_layout, sparsity_block_size,
                                        x.device, x.dtype, torch.is_grad_enabled(), w, b)
    if "sparsity_layout_w_t" not in layout_cache:
        layout_cache["sparsity_layout_w_t"] = _weight_layout(w, sparsity_block_size, x.device)
    layout_w_t = layout_cache["sparsity_layout_w_t"]
    if "w_t_bs" not in layout_cache:
        layout_cache["w_t_bs"] = _compress_weight(w, layout_w_t, sparsity_block_size)
    if "sparsity_layout_output" not in layout_cache:
        layout_cache["sparsity_layout_output"] = _output_layout(sparsity_layout, layout_w_t, b is not None)
    if b is not None and "bias_slice_bs" not in layout_cache:
        layout_cache["bias_slice_bs"] = _bias_blocks(b, sparsity_block_size)

    if "stacked_layouts" not in layout_cache:
        # the product's own cache is filed under the identity of its layouts, so these views are kept
        layout_cache["stacked_layouts"] = (_stack(sparsity_layout), _stack(layout_cache["sparsity_layout_output"]))
    stacked_layout, stacked_layout_output = layout_cache["stacked_layouts"]

    out = _project(x, stacked_layout, layout_cache["w_t_bs"], layout_w_t, stacked_layout_output,
                   layout_cache.get("bias_slice_bs"), sparsity_block_size,
                   layout_cache.setdefault("matmul_layout_cache", CacheHolder()).cache)
    layout_output = layout_cache["sparsity_layout_output"]
    finalize_layout_cache(layout_cache)
    return out, layout_output


def apply_torch_normalisation(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                              normalisation: nn.Module) -> BlksprsTensor:
    """Applies a row-wise PyTorch normalisation module to a block-sparse tensor (block rows without blocks are
    left out, so every row the module sees is a row of the compressed tensor).

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        normalisation (nn.Module): The normalisation module to apply.

    Returns:
        BlksprsTensor: The normalised tensor in compressed form.
    """
    return apply_function_applicable_row_wise(x, sparsity_layout, sparsity_block_size, normalisation)


def apply_torch_dropout(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                        dropout: nn.Dropout) -> BlksprsTensor:
    """Applies a PyTorch dropout module to a block-sparse tensor.

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        dropout (nn.Dropout): The dropout module to apply.

    Returns:
        BlksprsTensor: The result in compressed form.
    """
    return apply_function_applicable_row_wise(x, sparsity_layout, sparsity_block_size, dropout)


def apply_function_applicable_row_wise(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int,
                                       function: Callable) -> BlksprsTensor:
    """Applies a callable to the packed rows of a block-sparse tensor.

    The block rows that hold a block are stacked into one ``(1, rows * sbs, C * sbs)`` tensor, inactive blocks as
    zeros.  The callable must keep that shape and the device and must not mix rows; it may return another
    supported dtype.

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        function (Callable): The row-wise callable to apply.

    Returns:
        BlksprsTensor: The result in compressed form.
    """
    from ..ops.conversion import to_dense, to_sparse
    x = ensure_contiguous(x)

    validate_dimensions(x)
    validate_contiguous(x)
    validate_device(x)
    validate_dtype_supported(x)
    validate_sparsity(sparsity_block_size, (x, sparsity_layout))
    validate_sparsity_block_size(sparsity_block_size, x)
    if not callable(function):
        raise TypeError("Row-wise function must be callable")

    layout_packed = _pack_rows(sparsity_layout)
    pseudo_dense = to_dense(x, layout_packed, sparsity_block_size)
    result = function(pseudo_dense)
    if not isinstance(result, Tensor):
        raise TypeError("Row-wise function must return a Tensor")
    validate_shape(result, pseudo_dense.shape, "Row-wise function output")
    validate_device(result, pseudo_dense)
    validate_dtype_supported(result)
    return to_sparse(result, layout_packed, sparsity_block_size)


def _pack_rows(sparsity_layout: Tensor) -> Tensor:
    """The layout with the batch folded into the rows and the rows without blocks removed
    (blksprs/utils/processing.py:284-296); a layout without any block is only folded."""
    stacked = _stack(sparsity_layout)
    rows = torch.any(stacked != 0, dim=-1)
    if not torch.any(rows):
        return stacked
    return stacked[rows].unsqueeze(0)
