"""Construction of sparsity layouts."""

from .sparsity_layout import build_sparsity_layout, build_sparsity_layout_full, build_sparsity_layout_matmul

__all__ = ["build_sparsity_layout", "build_sparsity_layout_full", "build_sparsity_layout_matmul"]
