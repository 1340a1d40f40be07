"""MI355X-native block-sparse compute path with the blksprs operator interface.

``import blksprs_amd as bs`` gives ``bs.ops.matmul``, ``bs.ops.flash_attention``, ``bs.ops.softmax``,
``bs.ops.to_sparse`` / ``bs.ops.to_dense``, ``bs.layouting.build_sparsity_layout_matmul`` and the
validation switches under ``bs.utils`` with the reference's signatures; the work is done by hand-written
gfx950 HIP kernels in ``lib/libblksprs_amd.so``.
"""

import os as _os

# Accepted for import-time compatibility with the reference's BLKSPRS_AUTOTUNE switch
# (blksprs/utils/autotuning.py:5-9); tile shapes here are fixed per (block size, dtype) at compile time.
if _os.environ.get("BLKSPRS_AUTOTUNE", "DEFAULT").upper() not in ("DEFAULT", "TEST"):
    raise NotImplementedError(f"Unknown autotune mode: {_os.environ['BLKSPRS_AUTOTUNE']}")

from .utils.blksprs_tensor import BlksprsTensor

from . import layouting, ops, utils

__version__ = "0.1.0"

__all__ = ["BlksprsTensor", "layouting", "ops", "utils", "__version__"]
