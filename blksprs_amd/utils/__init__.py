"""Helpers shared by the block-sparse operators: validation switches, LUT builders, layout cache."""

from . import validation
from .tools import do_shape_blocksparse, undo_shape_blocksparse
from .validation import disable_contiguous, disable_validation, enable_contiguous, enable_validation

__all__ = [
    "disable_contiguous",
    "disable_validation",
    "do_shape_blocksparse",
    "enable_contiguous",
    "enable_validation",
    "undo_shape_blocksparse",
    "validation",
]
