"""Helpers shared by the block-sparse operators: validation switches, LUT builders, layout cache."""

from . import validation
from .processing import (apply_function_applicable_row_wise, apply_torch_dropout, apply_torch_linear,
                         apply_torch_linear_cached, apply_torch_normalisation)
from .tools import do_shape_blocksparse, undo_shape_blocksparse
from .validation import (disable_contiguous, disable_mask_facts, disable_validation, enable_contiguous,
                         enable_mask_facts, enable_validation, set_kept_ds_limit)

__all__ = [
    "apply_function_applicable_row_wise",
    "apply_torch_dropout",
    "apply_torch_linear",
    "apply_torch_linear_cached",
    "apply_torch_normalisation",
    "disable_contiguous",
    "disable_mask_facts",
    "disable_validation",
    "do_shape_blocksparse",
    "enable_contiguous",
    "enable_mask_facts",
    "enable_validation",
    "set_kept_ds_limit",
    "undo_shape_blocksparse",
    "validation",
]
