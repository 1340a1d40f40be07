"""Operations on compressed block-sparse tensors (the MI355X compute path)."""

from . import misc
from .conversion import from_blksprs, to_blksprs, to_dense, to_dense_shaped, to_sparse, to_sparse_shaped
from .flash_attention import flash_attention, flash_attention_build_layout_cache
from .matmul import matmul
from .softmax import softmax, softmax_fused, softmax_regular
from .transpose import transpose

__all__ = [
    "flash_attention",
    "flash_attention_build_layout_cache",
    "from_blksprs",
    "matmul",
    "misc",
    "softmax",
    "softmax_fused",
    "softmax_regular",
    "to_blksprs",
    "to_dense",
    "to_dense_shaped",
    "to_sparse",
    "to_sparse_shaped",
    "transpose",
]
