"""Helper operations without gradients (blksprs/ops/misc/__init__.py)."""

from .row_wise import row_wise_add, row_wise_max, row_wise_sub, row_wise_sum

__all__ = ["row_wise_add", "row_wise_max", "row_wise_sub", "row_wise_sum"]
