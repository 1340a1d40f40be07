"""Construction of sparsity layouts."""

from .causal import (build_causal_self_attention_layout, build_causal_self_attention_mask,
                     build_causal_window_self_attention_layout, build_causal_window_self_attention_mask)
from .sparsity_layout import (build_sparsity_layout, build_sparsity_layout_full, build_sparsity_layout_matmul,
                              build_sparsity_layout_matmul_fast, build_sparsity_layout_matmul_outer)

__all__ = ["build_causal_self_attention_layout", "build_causal_self_attention_mask",
           "build_causal_window_self_attention_layout", "build_causal_window_self_attention_mask",
           "build_sparsity_layout", "build_sparsity_layout_full", "build_sparsity_layout_matmul",
           "build_sparsity_layout_matmul_fast", "build_sparsity_layout_matmul_outer"]
