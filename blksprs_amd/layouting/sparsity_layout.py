"""Layout builders.

``build_sparsity_layout`` (the layout of a dense tensor: reference blksprs/layouting/sparsity_layout.py:17-109),
``build_sparsity_layout_full`` (:322-337) and the exact block product ``build_sparsity_layout_matmul``, the
default output layout of both ``matmul`` callers and ``flash_attention`` (:244-258, including the argument
checks of ``_validate_sparsity_layout_matmul_inputs``).  The two that look at data run on the device.
"""

import torch
from torch import Tensor

from .. import _capi
from ..utils.tools import layout_bytes, as_base_tensor
from ..utils.validation import (validate_contiguous, validate_device, validate_dimensions, validate_dtype_supported,
                                validate_sparsity_block_size, validate_sparsity_layout, _validation_enabled,
                                ensure_contiguous)


@torch.amp.custom_fwd(device_type="cuda")
def build_sparsity_layout(x: Tensor, sparsity_block_size: int) -> Tensor:
    """Builds the sparsity layout of a three-dimensional dense tensor.

    Args:
        x (Tensor): The dense tensor whose active blocks are represented by the layout.
        sparsity_block_size (int): The size of the sparsity blocks.

    Returns:
        Tensor: A Boolean sparsity layout marking every block containing a non-zero or NaN value.

    """
    x = ensure_contiguous(x)
    validate_dimensions(x)
    validate_contiguous(x)
    validate_device(x)
    validate_dtype_supported(x)
    validate_sparsity_block_size(sparsity_block_size, x)
    B, R, C = x.size(0), x.size(1) // sparsity_block_size, x.size(2) // sparsity_block_size
    out = torch.zeros((B, R, C), dtype=torch.bool, device=x.device)
    if out.numel():
        with torch.no_grad(), torch.cuda.device(x.device):
            _capi.call("bsa_layout_from_dense", _capi.ptr(x.detach()), out.view(torch.uint8).data_ptr(), B, R, C,
                       sparsity_block_size, x.element_size(), int(x.dtype.is_floating_point), _capi.stream(x.device))
    return as_base_tensor(out)


def build_sparsity_layout_full(x: Tensor, sparsity_block_size: int) -> Tensor:
    """Builds a fully populated sparsity layout for a dense tensor.

    Args:
        x (Tensor): A three-dimensional dense tensor.
        sparsity_block_size (int): The size of the sparsity blocks.

    Returns:
        Tensor: A boolean sparsity layout in which every block is active.

    """
    validate_dimensions(x)
    validate_device(x)
    validate_sparsity_block_size(sparsity_block_size, x)
    return torch.ones(size=(x.size(0), x.size(1) // sparsity_block_size, x.size(2) // sparsity_block_size),
                      dtype=torch.bool, device=x.device)


def _check_product_inputs(sparsity_layout_x: Tensor, sparsity_layout_y: Tensor) -> None:
    validate_dimensions(sparsity_layout_x, sparsity_layout_y)
    validate_contiguous(sparsity_layout_x, sparsity_layout_y)
    validate_device(sparsity_layout_x, sparsity_layout_y)
    validate_sparsity_layout(sparsity_layout_x, sparsity_layout_y)
    if not _validation_enabled():
        return
    if sparsity_layout_x.size(0) != sparsity_layout_y.size(0):
        raise ValueError("Batch dimensions of sparsity layouts must match")
    if sparsity_layout_x.size(-1) != sparsity_layout_y.size(-2):
        raise ValueError("Inner dimensions of sparsity layouts must match")


@torch.amp.custom_fwd(device_type="cuda")
def build_sparsity_layout_matmul(sparsity_layout_x: Tensor, sparsity_layout_y: Tensor) -> Tensor:
    """Builds the exact structural layout of a block-sparse matrix product.

    Args:
        sparsity_layout_x (Tensor): Layout of the left operand, ``(B, R, K)``.
        sparsity_layout_y (Tensor): Layout of the right operand, ``(B, K, C)``.

    Returns:
        Tensor: bool ``(B, R, C)`` layout, true where at least one ``k`` has both operand blocks active.

    """
    sparsity_layout_x, sparsity_layout_y = ensure_contiguous(sparsity_layout_x, sparsity_layout_y)
    _check_product_inputs(sparsity_layout_x, sparsity_layout_y)
    B, R, K = sparsity_layout_x.shape
    C = sparsity_layout_y.size(2)
    dev = sparsity_layout_x.device
    out = torch.empty((B, R, C), dtype=torch.bool, device=dev)
    if out.numel():
        lx, ly = layout_bytes(sparsity_layout_x), layout_bytes(sparsity_layout_y)
        with _capi.on_device(dev):
            _capi.call("bsa_layout_matmul", _capi.ptr(lx), _capi.ptr(ly), B, R, K, C,
                       out.view(torch.uint8).data_ptr(), _capi.stream(dev))
    return as_base_tensor(out)


def _row_and_column_activity(sparsity_layout_x: Tensor, sparsity_layout_y: Tensor) -> tuple[Tensor, Tensor]:
    """``(B, R, 1)`` rows of x and ``(B, 1, C)`` columns of y that hold a block."""
    _check_product_inputs(sparsity_layout_x, sparsity_layout_y)
    rows = torch.any(as_base_tensor(sparsity_layout_x) != 0, dim=-1, keepdim=True)
    columns = torch.any(as_base_tensor(sparsity_layout_y) != 0, dim=-2, keepdim=True)
    return rows, columns


@torch.amp.custom_fwd(device_type="cuda")
def build_sparsity_layout_matmul_fast(sparsity_layout_x: Tensor, sparsity_layout_y: Tensor) -> Tensor:
    """Conservative product layout: block ``(i, j)`` is active when row ``i`` of x AND column ``j`` of y hold a
    block, whether or not they meet at one ``k`` (blksprs/layouting/sparsity_layout.py:262-283).  A superset
    of :func:`build_sparsity_layout_matmul`.

    Args:
        sparsity_layout_x (Tensor): Layout of the left operand, ``(B, R, K)``.
        sparsity_layout_y (Tensor): Layout of the right operand, ``(B, K, C)``.

    Returns:
        Tensor: bool ``(B, R, C)`` layout.
    """
    rows, columns = _row_and_column_activity(sparsity_layout_x, sparsity_layout_y)
    return as_base_tensor(torch.logical_and(rows, columns))


@torch.amp.custom_fwd(device_type="cuda")
def build_sparsity_layout_matmul_outer(sparsity_layout_x: Tensor, sparsity_layout_y: Tensor) -> Tensor:
    """Outer product layout: block ``(i, j)`` is active when row ``i`` of x OR column ``j`` of y holds a block
    (blksprs/layouting/sparsity_layout.py:286-311); for products followed by something that fills more
    blocks, such as a bias.

    Args:
        sparsity_layout_x (Tensor): Layout of the left operand, ``(B, R, K)``.
        sparsity_layout_y (Tensor): Layout of the right operand, ``(B, K, C)``.

    Returns:
        Tensor: bool ``(B, R, C)`` layout.
    """
    rows, columns = _row_and_column_activity(sparsity_layout_x, sparsity_layout_y)
    return as_base_tensor(torch.logical_or(rows, columns))
