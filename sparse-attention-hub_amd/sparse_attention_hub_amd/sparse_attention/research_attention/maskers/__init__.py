"""Masker plug-ins of ResearchAttention."""
from .base import AttentionTensorDimensions, MaskerConfig, MaskerRegistry, ResearchMasker
from .fixed import (  # noqa: F401  (importing registers the maskers)
    CausalMasker, FixedMasker, FixedMaskerConfig, HashAttentionTopKMasker, HashAttentionTopKMaskerConfig,
    LocalMasker, LocalMaskerConfig, OracleTopK, OracleTopKConfig, PQCache, PQCacheConfig, SinkMasker,
    SinkMaskerConfig, TopKMasker, TopKMaskerConfig,
)
from .sampling import (  # noqa: F401
    AdaptiveSamplingMasker, AdaptiveSamplingMaskerConfig, RandomSamplingMasker, RandomSamplingMaskerConfig,
    SamplingMasker, SamplingMaskerConfig,
)

__all__ = ["AttentionTensorDimensions", "MaskerConfig", "MaskerRegistry", "ResearchMasker"]
