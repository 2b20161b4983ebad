"""MI355X-native ResearchAttention decode path (sparse-attention-hub API on HIP kernels)."""
from .sparse_attention import (  # noqa: F401
    Mask, ResearchAttention, ResearchAttentionConfig, SparseAttention, SparseAttentionConfig,
)

__all__ = ["Mask", "ResearchAttention", "ResearchAttentionConfig", "SparseAttention", "SparseAttentionConfig"]
__version__ = "0.1.0"
