"""Transposition of a compressed block-sparse tensor.

Same signature, cache keys and gradient as the reference (blksprs/ops/transpose.py:13-98).  The reference
transposes the elements of every block with torch and then gathers the blocks with ``flow_pull_kernel``
(blksprs/ops/flow.py:11-111); here one kernel (``bsa_transpose_blocks``) does both.
"""

import torch
from torch import Tensor

from .. import _capi
from ..utils.blksprs_tensor import BlksprsTensor
from ..utils.tools import (as_base_tensor, eager_only, finalize_layout_cache, nonzero_from_packed, pack_layouts,
                           prepare_layout_cache)
from ..utils.validation import (ensure_contiguous, validate_contiguous, validate_device, validate_dimensions,
                                validate_dtype_supported, validate_sparsity, validate_sparsity_block_size)


def _launch(x: Tensor, sparsity_layout_t: Tensor, layout_indices: Tensor, packed_indices: Tensor, sbs: int,
            n_sparse_blocks: int) -> Tensor:
    out = torch.empty((n_sparse_blocks, sbs, sbs), dtype=x.dtype, device=x.device)
    if n_sparse_blocks:
        B, R, C = (int(s) for s in sparsity_layout_t.shape)
        with _capi.on_device(x.device):
            _capi.call("bsa_transpose_blocks", _capi.ptr(x), layout_indices.data_ptr(), packed_indices.data_ptr(),
                       out.data_ptr(), n_sparse_blocks, x.size(0), B, R, C, sbs, x.element_size(),
                       _capi.stream(x.device))
    return out


class _Transpose(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, sparsity_layout_t, layout_indices, packed_indices, sparsity_block_size, n_sparse_blocks):
        ctx.save_for_backward(sparsity_layout_t)
        ctx.sparsity_block_size = sparsity_block_size
        return _launch(x, sparsity_layout_t, layout_indices, packed_indices, sparsity_block_size, n_sparse_blocks)

    @staticmethod
    def backward(ctx, grad_output):
        # the gradient is the transpose back: the transposed layout is the layout of grad_output
        (sparsity_layout_t,) = ctx.saved_tensors
        grad = transpose(grad_output.contiguous(), sparsity_layout_t, ctx.sparsity_block_size)[0]
        return grad, None, None, None, None, None


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def transpose(x: BlksprsTensor, sparsity_layout: Tensor,
              sparsity_block_size: int, layout_cache: dict | None = None) -> tuple[BlksprsTensor, Tensor]:
    """Transposes a block-sparse tensor in compressed form.

    Args:
        x (BlksprsTensor): The compressed input tensor.
        sparsity_layout (Tensor): The sparsity layout of ``x``.
        sparsity_block_size (int): The size of the sparsity blocks.
        layout_cache (dict, optional): Reusable layout metadata cache (default ``None``).

    Returns:
        tuple[BlksprsTensor, Tensor]: The transposed tensor in compressed form and its sparsity layout.

    """
    x = ensure_contiguous(x)

    validate_dimensions(x)
    validate_contiguous(x)
    validate_dtype_supported(x)
    validate_device(x)
    validate_sparsity(sparsity_block_size, (x, sparsity_layout))
    validate_sparsity_block_size(sparsity_block_size, x)

    layout_cache = transpose_build_layout_cache(layout_cache, sparsity_layout)

    out = _Transpose.apply(x, layout_cache["sparsity_layout_t"], layout_cache["layout_indices"],
                           layout_cache["packed_indices"], sparsity_block_size, layout_cache["n_sparse_blocks"])
    return BlksprsTensor.wrap(out), layout_cache["sparsity_layout_t"]


def transpose_build_layout_cache(layout_cache: dict | None, sparsity_layout: Tensor) -> dict:
    """Metadata of one layout: ``sparsity_layout_t`` (the transposed layout, own storage), ``layout_indices``
    (its non-zero coordinates), ``packed_indices`` (the packed indices of ``sparsity_layout`` arranged in
    transposed order: the source block of every position of the transposed layout) and ``n_sparse_blocks``."""
    layout_cache = prepare_layout_cache(layout_cache, "transpose", sparsity_layout)

    if "sparsity_layout_t" not in layout_cache:
        sparsity_layout_t = as_base_tensor(sparsity_layout.transpose(-1, -2).contiguous())
        if sparsity_layout_t.data_ptr() == sparsity_layout.data_ptr():
            sparsity_layout_t = sparsity_layout_t.clone()
        layout_cache["sparsity_layout_t"] = sparsity_layout_t

    need_packed = "packed_indices" not in layout_cache or "n_sparse_blocks" not in layout_cache
    need_indices = "layout_indices" not in layout_cache
    if need_packed or need_indices:
        # both scans in one batch: their counts come back in one read
        specs = ([(sparsity_layout, 0)] if need_packed else []) + \
                ([(layout_cache["sparsity_layout_t"], 0)] if need_indices else [])
        infos = pack_layouts(*specs)
        if need_packed:
            info = infos[0]
            layout_cache["packed_indices"] = (info.packed.reshape(sparsity_layout.size())
                                              .transpose(-1, -2).contiguous().reshape(-1))
            layout_cache["n_sparse_blocks"] = info.count
        if need_indices:
            info_t = infos[-1]
            layout_cache["layout_indices"] = nonzero_from_packed(info_t.packed,
                                                                 layout_cache["sparsity_layout_t"].shape, info_t.count)

    validate_contiguous(layout_cache["sparsity_layout_t"], layout_cache["layout_indices"],
                        layout_cache["packed_indices"])

    return finalize_layout_cache(layout_cache)
