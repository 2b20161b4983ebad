"""Sampling masker implementations."""
from .adaptive_sampling import AdaptiveSamplingMasker, AdaptiveSamplingMaskerConfig

__all__ = ["AdaptiveSamplingMasker", "AdaptiveSamplingMaskerConfig"]
