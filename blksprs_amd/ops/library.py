"""The primitive operators as ``torch.library`` operators (namespace ``blksprs_amd``).

The reference registers its kernel launchers as ``blksprs::matmul_forward``, ``to_sparse_forward``,
``to_dense_forward``, ``softmax_fused_forward`` and ``softmax_fused_backward`` (``blksprs/ops/matmul.py:70``,
``blksprs/ops/conversion.py:191``, ``:463``, ``blksprs/ops/softmax.py:437``, ``:478``), each a function of the
operands, the lookup tables of the layout cache and the block size that returns a fresh tensor and mutates
nothing.  The operators here are the same launchers of this library under their own namespace (the two
packages can be imported side by side), with the tables this library's kernels walk in place of the
reference's, and with shape functions, so that they can be traced with fake tensors.  The public wrappers
(``bs.ops.matmul`` ...) call the launchers directly: going through the dispatcher costs several microseconds
per call and buys nothing in eager mode, which is the only mode the wrappers run in (they are marked
``torch.compiler.disable``, as the reference's are graph breaks).

    out = torch.ops.blksprs_amd.matmul_forward(x, y, cache["contraction_offsets"], cache["contraction_pairs"],
                                               cache["n_sparse_blocks"], 64, False, False)
"""

import torch
from torch import Tensor

from .. import _capi

_NAMESPACE = "blksprs_amd"


def _register(name: str, launcher, shape_function) -> None:
    operator = torch.library.custom_op(f"{_NAMESPACE}::{name}", launcher, mutates_args=(), device_types="cuda")
    operator.register_fake(shape_function)


def _matmul_forward(x: Tensor, y: Tensor, contraction_offsets: Tensor, contraction_pairs: Tensor,
                    n_sparse_blocks: int, sparsity_block_size: int, transpose_x: bool, transpose_y: bool) -> Tensor:
    from .matmul import _launch
    return _launch(x, y, contraction_offsets, contraction_pairs, None, n_sparse_blocks, sparsity_block_size,
                   transpose_x, transpose_y)


def _matmul_shape(x, y, contraction_offsets, contraction_pairs, n_sparse_blocks, sparsity_block_size, transpose_x,
                  transpose_y):
    return x.new_empty((n_sparse_blocks, sparsity_block_size, sparsity_block_size))


def _to_sparse_forward(x: Tensor, layout_indices: Tensor, sparsity_block_size: int, n_sparse_blocks: int) -> Tensor:
    from .conversion import _launch_to_sparse
    return _launch_to_sparse(x, layout_indices, sparsity_block_size, n_sparse_blocks)


def _to_sparse_shape(x, layout_indices, sparsity_block_size, n_sparse_blocks):
    return x.new_empty((n_sparse_blocks, sparsity_block_size, sparsity_block_size))


def _to_dense_forward(x: Tensor, sparsity_layout: Tensor, packed_indices: Tensor, sparsity_block_size: int,
                      fill_value: float) -> Tensor:
    from .conversion import _launch_to_dense
    return _launch_to_dense(x, sparsity_layout.shape, packed_indices, sparsity_block_size, fill_value)


def _to_dense_shape(x, sparsity_layout, packed_indices, sparsity_block_size, fill_value):
    return x.new_empty((sparsity_layout.size(0), sparsity_layout.size(1) * sparsity_block_size,
                        sparsity_layout.size(2) * sparsity_block_size))


def _softmax_fused_forward(x: Tensor, row_offsets: Tensor, n_rows: int, sparsity_block_size: int) -> Tensor:
    out = torch.empty_like(x)
    with _capi.on_device(x.device):
        _capi.call("bsa_softmax_fwd", x.data_ptr(), out.data_ptr(), row_offsets.data_ptr(), n_rows, x.size(0),
                   sparsity_block_size, _capi.stream(x.device))
    return out


def _softmax_fused_backward(grad_output: Tensor, o: Tensor, row_offsets: Tensor, n_rows: int,
                            sparsity_block_size: int) -> Tensor:
    grad_x = torch.empty_like(o)
    with _capi.on_device(o.device):
        _capi.call("bsa_softmax_bwd", grad_output.data_ptr(), o.data_ptr(), grad_x.data_ptr(),
                   row_offsets.data_ptr(), n_rows, o.size(0), sparsity_block_size, _capi.stream(o.device))
    return grad_x


_register("matmul_forward", _matmul_forward, _matmul_shape)
_register("to_sparse_forward", _to_sparse_forward, _to_sparse_shape)
_register("to_dense_forward", _to_dense_forward, _to_dense_shape)
_register("softmax_fused_forward", _softmax_fused_forward, lambda x, row_offsets, n_rows, sbs: torch.empty_like(x))
_register("softmax_fused_backward", _softmax_fused_backward,
          lambda grad_output, o, row_offsets, n_rows, sbs: torch.empty_like(o))
