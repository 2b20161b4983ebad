"""Sampling maskers."""
from .base import SamplingMasker, SamplingMaskerConfig
from .implementations import (
    AdaptiveSamplingMasker, AdaptiveSamplingMaskerConfig, RandomSamplingMasker, RandomSamplingMaskerConfig,
)

__all__ = ["SamplingMasker", "SamplingMaskerConfig", "AdaptiveSamplingMasker", "AdaptiveSamplingMaskerConfig",
           "RandomSamplingMasker", "RandomSamplingMaskerConfig"]
