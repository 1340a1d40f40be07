"""Marker type for compressed block-sparse tensors.

Mirrors the behaviour of the reference's ``BlksprsTensor``
(blksprs/utils/blksprs_tensor.py:7-25): a ``torch.Tensor`` subclass with no
extra state whose only job is to tag a ``(n_blocks, sbs, sbs)`` tensor as
"compressed".  Operators return it; tests assert on the type.
"""

import torch
from torch import Tensor


class BlksprsTensor(Tensor):
    """A ``(n_sparse_blocks, sbs, sbs)`` tensor holding only the active blocks of a layout."""

    def __repr__(self, *, tensor_contents=None):
        inner = Tensor.__repr__(Tensor(self), tensor_contents=tensor_contents)
        return "BlksprsTensor(" + inner + ")"

    @staticmethod
    def wrap(tensor: Tensor) -> "BlksprsTensor":
        # Tensor subclasses cannot be constructed while Dynamo traces a frame;
        # the compressed representation is identical either way.
        if torch._dynamo.is_compiling():
            return tensor  # type: ignore[return-value]
        return BlksprsTensor(tensor)
