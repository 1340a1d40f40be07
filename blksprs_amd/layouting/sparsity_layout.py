"""Structural layout builders.

Only the exact block product is built here, on the device, because the product
layout is the default output layout of both ``matmul`` callers and
``flash_attention`` (reference: blksprs/layouting/sparsity_layout.py:244-258,
including the argument checks of ``_validate_sparsity_layout_matmul_inputs``).
"""

import torch
from torch import Tensor

from .. import _capi
from ..utils.tools import _layout_bytes, as_base_tensor
from ..utils.validation import (validate_contiguous, validate_device, validate_dimensions,
                                validate_sparsity_layout, _validation_enabled, ensure_contiguous)


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
        lx, ly = _layout_bytes(sparsity_layout_x), _layout_bytes(sparsity_layout_y)
        with torch.cuda.device(dev):
            _capi.call("bsa_layout_matmul", _capi.ptr(lx), _capi.ptr(ly), B, R, K, C,
                       out.view(torch.uint8).data_ptr(), _capi.stream(dev))
    return as_base_tensor(out)
