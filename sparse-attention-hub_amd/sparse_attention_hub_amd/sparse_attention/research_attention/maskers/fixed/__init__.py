"""Fixed-pattern and top-k maskers."""
from .base import FixedMasker, FixedMaskerConfig, TopKMasker, TopKMaskerConfig, TopPMaskerConfig
from .implementations import (
    CausalMasker, HashAttentionTopKMasker, HashAttentionTopKMaskerConfig, LocalMasker, LocalMaskerConfig,
    OracleTopK, OracleTopKConfig, PQCache, PQCacheConfig, SinkMasker, SinkMaskerConfig,
)

__all__ = [
    "FixedMasker", "FixedMaskerConfig", "TopKMasker", "TopKMaskerConfig", "TopPMaskerConfig",
    "CausalMasker", "LocalMasker", "LocalMaskerConfig", "SinkMasker", "SinkMaskerConfig",
    "OracleTopK", "OracleTopKConfig", "HashAttentionTopKMasker", "HashAttentionTopKMaskerConfig",
    "PQCache", "PQCacheConfig",
]
