"""Sampling maskers."""
from .base import SamplingMasker, SamplingMaskerConfig
from .implementations import AdaptiveSamplingMasker, AdaptiveSamplingMaskerConfig

__all__ = ["SamplingMasker", "SamplingMaskerConfig", "AdaptiveSamplingMasker", "AdaptiveSamplingMaskerConfig"]
