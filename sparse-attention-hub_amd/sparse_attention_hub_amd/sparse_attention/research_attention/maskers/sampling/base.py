"""Sampling masker base (reference: maskers/sampling/base.py:13-48)."""
from __future__ import annotations

from dataclasses import dataclass

from ..base import MaskerConfig, ResearchMasker


@dataclass
class SamplingMaskerConfig(MaskerConfig):
    """Base configuration for sampling maskers."""


class SamplingMasker(ResearchMasker):
    def __init__(self, config: SamplingMaskerConfig) -> None:
        super().__init__(config)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "SamplingMasker":
        if not isinstance(config, SamplingMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)
