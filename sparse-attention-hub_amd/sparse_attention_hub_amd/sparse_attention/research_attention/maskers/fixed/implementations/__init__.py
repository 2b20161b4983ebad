"""Concrete fixed / top-k maskers (importing this package registers them)."""
from .basic_fixed import CausalMasker, LocalMasker, LocalMaskerConfig, SinkMasker, SinkMaskerConfig
from .hashattention_top_k import HashAttentionTopKMasker, HashAttentionTopKMaskerConfig
from .oracle_top_k import OracleTopK, OracleTopKConfig
from .pq_top_k import PQCache, PQCacheConfig

__all__ = [
    "CausalMasker", "LocalMasker", "LocalMaskerConfig", "SinkMasker", "SinkMaskerConfig",
    "OracleTopK", "OracleTopKConfig", "HashAttentionTopKMasker", "HashAttentionTopKMaskerConfig",
    "PQCache", "PQCacheConfig",
]
