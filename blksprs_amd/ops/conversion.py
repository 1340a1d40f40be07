"""Dense <-> compressed conversion.

Same signatures, cache keys and aliasing rules as the reference
(blksprs/ops/conversion.py:17-55, :158-304, :307-348, :429-621); the copies are
done by ``bsa_to_sparse`` / ``bsa_to_dense``.
"""

import torch
from torch import Tensor

from .. import _capi
from ..utils.blksprs_tensor import BlksprsTensor
from ..utils.tools import (eager_only, finalize_layout_cache, nonzero_from_packed, pack_layout, prepare_layout_cache)
from ..utils.validation import (ensure_contiguous, validate_contiguous, validate_device, validate_dimensions,
                                validate_dtype_supported, validate_sparsity, validate_sparsity_block_size,
                                validate_sparsity_dense)


def _fill_bits(fill_value, dtype: torch.dtype) -> int:
    """Bit pattern of ``fill_value`` converted to ``dtype`` the way ``torch.full`` converts it."""
    scalar = torch.full((1,), fill_value, dtype=dtype)
    width = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[scalar.element_size()]
    return int(scalar.view(width).item()) & ((1 << (8 * scalar.element_size())) - 1)


def _single_full_block(sparsity_layout: Tensor) -> bool:
    return sparsity_layout.size(1) == 1 and sparsity_layout.size(2) == 1 and bool(torch.all(sparsity_layout))


def _launch_to_sparse(x: Tensor, layout_indices: Tensor, sbs: int, n_sparse_blocks: int) -> Tensor:
    out = torch.empty((n_sparse_blocks, sbs, sbs), dtype=x.dtype, device=x.device)
    if n_sparse_blocks:
        with _capi.on_device(x.device):
            _capi.call("bsa_to_sparse", x.data_ptr(), layout_indices.data_ptr(), out.data_ptr(), n_sparse_blocks,
                       x.size(1), x.size(2), sbs, x.element_size(), _capi.stream(x.device))
    return out


def _launch_to_dense(x: Tensor, shape, packed_indices: Tensor, sbs: int, fill_value) -> Tensor:
    B, R, C = (int(s) for s in shape)
    out = torch.empty((B, R * sbs, C * sbs), dtype=x.dtype, device=x.device)
    if out.numel():
        with _capi.on_device(x.device):
            _capi.call("bsa_to_dense", _capi.ptr(x), packed_indices.data_ptr(), out.data_ptr(), B, R, C, x.size(0),
                       sbs, x.element_size(), _fill_bits(fill_value, x.dtype), _capi.stream(x.device))
    return out


class _ToSparse(torch.autograd.Function):
    # The layout is metadata, not a differentiable input: it is kept as a plain attribute, so that a compressed
    # tensor held in a cache (the packed weight of apply_torch_linear_cached) can be differentiated through in
    # every training iteration, not only in the first.
    @staticmethod
    def forward(ctx, x, sparsity_layout, layout_indices, sparsity_block_size, n_sparse_blocks):
        ctx.sparsity_layout = sparsity_layout
        ctx.sparsity_block_size = sparsity_block_size
        return _launch_to_sparse(x, layout_indices, sparsity_block_size, n_sparse_blocks)

    @staticmethod
    def backward(ctx, grad_output):
        sparsity_layout = ctx.sparsity_layout
        grad = to_dense(grad_output.contiguous(), sparsity_layout, ctx.sparsity_block_size)
        return grad, None, None, None, None


class _ToDense(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, sparsity_layout, packed_indices, sparsity_block_size, fill_value):
        ctx.sparsity_layout = sparsity_layout
        ctx.sparsity_block_size = sparsity_block_size
        return _launch_to_dense(x, sparsity_layout.shape, packed_indices, sparsity_block_size, fill_value)

    @staticmethod
    def backward(ctx, grad_output):
        sparsity_layout = ctx.sparsity_layout
        grad = to_sparse(grad_output.contiguous(), sparsity_layout, ctx.sparsity_block_size)
        return grad, None, None, None, None


def to_sparse_build_layout_cache(layout_cache: dict | None, sparsity_layout: Tensor) -> dict:
    layout_cache = prepare_layout_cache(layout_cache, "to_sparse", sparsity_layout)
    if "layout_indices" not in layout_cache or "n_sparse_blocks" not in layout_cache:
        info = pack_layout(sparsity_layout)
        layout_cache["layout_indices"] = nonzero_from_packed(info.packed, sparsity_layout.shape, info.count)
        layout_cache["n_sparse_blocks"] = info.count
    validate_contiguous(sparsity_layout, layout_cache["layout_indices"])
    return finalize_layout_cache(layout_cache)


def to_dense_build_layout_cache(layout_cache: dict | None, sparsity_layout: Tensor) -> dict:
    layout_cache = prepare_layout_cache(layout_cache, "to_dense", sparsity_layout)
    if "packed_indices" not in layout_cache:
        layout_cache["packed_indices"] = pack_layout(sparsity_layout).packed
    validate_contiguous(layout_cache["packed_indices"])
    return finalize_layout_cache(layout_cache)


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def to_sparse(x: Tensor, sparsity_layout: Tensor,
              sparsity_block_size: int, layout_cache: dict | None = None) -> BlksprsTensor:
    """Converts a three-dimensional dense tensor to compressed block-sparse form.

    Args:
        x (Tensor): The dense input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        layout_cache (dict, optional): Reusable layout metadata cache (default ``None``).

    Returns:
        BlksprsTensor: ``x`` in compressed form.

    """
    x = ensure_contiguous(x)

    validate_dimensions(x)
    validate_contiguous(x)
    validate_device(x)
    validate_dtype_supported(x)
    validate_sparsity_dense(sparsity_block_size, (x, sparsity_layout))
    validate_sparsity_block_size(sparsity_block_size, x)

    layout_cache = to_sparse_build_layout_cache(layout_cache, sparsity_layout)

    # a single all-active block is its own compressed form: hand the storage back
    if _single_full_block(sparsity_layout):
        return BlksprsTensor.wrap(x)

    return BlksprsTensor.wrap(_ToSparse.apply(x, sparsity_layout, layout_cache["layout_indices"],
                                              sparsity_block_size, layout_cache["n_sparse_blocks"]))


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def to_dense(x: BlksprsTensor, sparsity_layout: Tensor,
             sparsity_block_size: int, fill_value: float = 0, layout_cache: dict | None = None) -> Tensor:
    """Converts a compressed block-sparse tensor to three-dimensional dense form.

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        fill_value (float, optional): The value used for inactive blocks (default ``0``).
        layout_cache (dict, optional): Reusable layout metadata cache (default ``None``).

    Returns:
        Tensor: ``x`` in three-dimensional dense form.

    """
    x = ensure_contiguous(x)

    validate_dimensions(x)
    validate_contiguous(x, sparsity_layout)
    validate_device(x)
    validate_dtype_supported(x)
    validate_sparsity(sparsity_block_size, (x, sparsity_layout))
    validate_sparsity_block_size(sparsity_block_size, x)

    layout_cache = to_dense_build_layout_cache(layout_cache, sparsity_layout)

    if _single_full_block(sparsity_layout):
        return Tensor(x)

    return Tensor(_ToDense.apply(x, sparsity_layout, layout_cache["packed_indices"], sparsity_block_size,
                                 fill_value))


def to_blksprs(x: Tensor, sparsity_layout: Tensor, sparsity_block_size: int,
               layout_cache: dict | None = None) -> BlksprsTensor:
    """Alias of :func:`to_sparse`."""
    return to_sparse(x, sparsity_layout, sparsity_block_size, layout_cache=layout_cache)


def to_sparse_shaped(x: Tensor, sparsity_layout: Tensor, sparsity_block_size: int,
                     layout_cache: dict | None = None) -> BlksprsTensor:
    """Alias of :func:`to_sparse` for inputs that already have shape ``(B, rows, cols)``."""
    return to_sparse(x, sparsity_layout, sparsity_block_size, layout_cache=layout_cache)


def from_blksprs(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int, fill_value: float = 0,
                 layout_cache: dict | None = None) -> Tensor:
    """Alias of :func:`to_dense`."""
    return to_dense(x, sparsity_layout, sparsity_block_size, fill_value=fill_value, layout_cache=layout_cache)


def to_dense_shaped(x: BlksprsTensor, sparsity_layout: Tensor, sparsity_block_size: int, fill_value: float = 0,
                    layout_cache: dict | None = None) -> Tensor:
    """Alias of :func:`to_dense` whose result keeps shape ``(B, rows, cols)``."""
    return to_dense(x, sparsity_layout, sparsity_block_size, fill_value=fill_value, layout_cache=layout_cache)
