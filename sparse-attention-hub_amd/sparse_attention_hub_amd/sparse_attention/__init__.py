"""Sparse attention: the ResearchAttention decode path on MI355X kernels."""
from .base import SparseAttention, SparseAttentionConfig
from .research_attention import ResearchAttention, ResearchAttentionConfig
from .research_attention.maskers import MaskerConfig, MaskerRegistry, ResearchMasker
from .research_attention.maskers.fixed import (
    CausalMasker, FixedMasker, FixedMaskerConfig, HashAttentionTopKMasker, HashAttentionTopKMaskerConfig,
    LocalMasker, LocalMaskerConfig, OracleTopK, OracleTopKConfig, PQCache, PQCacheConfig, SinkMasker,
    SinkMaskerConfig, TopKMasker, TopKMaskerConfig,
)
from .research_attention.maskers.sampling import (
    AdaptiveSamplingMasker, AdaptiveSamplingMaskerConfig, RandomSamplingMasker, RandomSamplingMaskerConfig,
    SamplingMasker, SamplingMaskerConfig,
)
from .utils.mask import Mask

__all__ = [
    "SparseAttention", "SparseAttentionConfig", "ResearchAttention", "ResearchAttentionConfig",
    "MaskerConfig", "MaskerRegistry", "ResearchMasker",
    "FixedMasker", "FixedMaskerConfig", "TopKMasker", "TopKMaskerConfig",
    "CausalMasker", "LocalMasker", "LocalMaskerConfig", "SinkMasker", "SinkMaskerConfig",
    "OracleTopK", "OracleTopKConfig", "HashAttentionTopKMasker", "HashAttentionTopKMaskerConfig",
    "PQCache", "PQCacheConfig", "SamplingMasker", "SamplingMaskerConfig",
    "AdaptiveSamplingMasker", "AdaptiveSamplingMaskerConfig", "RandomSamplingMasker", "RandomSamplingMaskerConfig",
    "Mask",
]
