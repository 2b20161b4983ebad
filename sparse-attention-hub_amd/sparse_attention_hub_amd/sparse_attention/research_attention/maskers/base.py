"""Masker plug-in contract (reference: research_attention/maskers/base.py:16-208).

A masker is built from a config dataclass through `MaskerRegistry` and adds its
selection to the mask it is handed: `add_mask(..., previous_mask) -> Mask`.
The concrete maskers of this package keep the mask in the kernels' row layout
and extend it in place with one or two HIP launches.
"""
from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple, Type, TypeVar, Union

import torch

from ...utils.mask import Mask

T = TypeVar("T", bound="ResearchMasker")
ConfigType = TypeVar("ConfigType", bound="MaskerConfig")


@dataclass
class MaskerConfig:
    """Base configuration class for all maskers."""


@dataclass
class AttentionTensorDimensions:
    batch_size: int
    num_heads: int
    seq_len_queries: int
    seq_len_keys: int


class MaskerRegistry:
    """config class -> masker class, filled by the `register` decorator."""

    _registry: Dict[Type[MaskerConfig], Type["ResearchMasker"]] = {}

    @classmethod
    def register(cls, config_type: Type[ConfigType]) -> Callable[[Type[T]], Type[T]]:
        def decorator(masker_class: Type[T]) -> Type[T]:
            cls._registry[config_type] = masker_class
            return masker_class

        return decorator

    @classmethod
    def get_masker_class(cls, config_type: Type[MaskerConfig]) -> Type["ResearchMasker"]:
        masker_class = cls._registry.get(config_type)
        if masker_class is None:
            raise ValueError(f"No masker class registered for config type: {config_type}")
        return masker_class

    @classmethod
    def get_all_registered_types(cls) -> Dict[Type[MaskerConfig], Type["ResearchMasker"]]:
        return cls._registry.copy()


class ResearchMasker(ABC):
    config: MaskerConfig

    def __init__(self, config: MaskerConfig) -> None:
        self.config = config

    def _extract_tensor_dimensions(self, keys: torch.Tensor, queries: torch.Tensor) -> AttentionTensorDimensions:
        # heads are the *query* heads: mask rows are per query head
        return AttentionTensorDimensions(
            batch_size=queries.shape[0],
            num_heads=queries.shape[1],
            seq_len_queries=queries.shape[2],
            seq_len_keys=keys.shape[2],
        )

    @staticmethod
    def _mask_shape(dims: AttentionTensorDimensions) -> Tuple[int, int, int, int]:
        return (dims.batch_size, dims.num_heads, dims.seq_len_queries, dims.seq_len_keys)

    def _create_full_mask(self, dims: AttentionTensorDimensions, dtype: torch.dtype, device: torch.device) -> Mask:
        return Mask.create_full_mask(self._mask_shape(dims), dtype=dtype, device=device)

    def _create_mask_from_rowise_indices(
        self, dims: AttentionTensorDimensions, indices: torch.Tensor, device: torch.device, dtype: torch.dtype
    ) -> Mask:
        """Ones at the given per-row key indices (container utility, dense form)."""
        data = torch.ones_like(indices, dtype=dtype, device=device)
        return Mask.create_from_row_wise_idx(
            shape=self._mask_shape(dims), row_wise_idx=indices, data=data, mask_type="dense", dtype=dtype
        )

    def _calculate_effective_size(self, size_param: Union[float, int], seq_len_keys: int) -> int:
        """float = fraction of the keys (truncated), int = absolute."""
        if isinstance(size_param, float):
            return int(size_param * seq_len_keys)
        return int(size_param)

    @abstractmethod
    def add_mask(
        self,
        keys: torch.Tensor,
        queries: torch.Tensor,
        values: torch.Tensor,
        attention_mask: torch.Tensor,
        scaling: float,
        dropout: float,
        sparse_meta_data: Dict[Any, Any],
        previous_mask: Mask,
        **kwargs: Dict[str, Any],
    ) -> Mask:
        ...

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        """Upper bound of the entries this masker appends to a row, or None if it is
        only known on the device. Lets the caller size the row buffers once."""
        return None

    @classmethod
    @abstractmethod
    def create_from_config(cls, config: MaskerConfig) -> "ResearchMasker":
        ...

    @classmethod
    def create_masker_from_config(cls, config: MaskerConfig) -> "ResearchMasker":
        masker_class = MaskerRegistry.get_masker_class(type(config))
        return masker_class.create_from_config(config)
