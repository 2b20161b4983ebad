"""Sparse-attention base types (reference: sparse_attention/base.py:11-75)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

import torch
from torch import nn


@dataclass
class SparseAttentionConfig:
    """Configuration class for sparse attention mechanisms."""


class SparseAttention(ABC):
    sparse_attention_config: SparseAttentionConfig

    def __init__(self, sparse_attention_config: SparseAttentionConfig) -> None:
        self.sparse_attention_config = sparse_attention_config

    @abstractmethod
    def custom_attention(
        self,
        module: nn.Module,
        queries: torch.Tensor,
        keys: torch.Tensor,
        values: torch.Tensor,
        attention_mask: Optional[torch.Tensor],
        scaling: float,
        dropout: float,
        **kwargs: Dict[str, Any],
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        ...

    def pre_attention_hook_generator(self) -> None:
        return None

    @classmethod
    def create_from_config(cls, config: SparseAttentionConfig) -> "SparseAttention":
        """Route a config to the class that implements it."""
        from .research_attention import ResearchAttention, ResearchAttentionConfig

        if isinstance(config, ResearchAttentionConfig):
            return ResearchAttention.create_from_config(config)
        return cls(config)
