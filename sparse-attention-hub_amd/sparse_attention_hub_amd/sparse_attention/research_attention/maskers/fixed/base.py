"""Fixed-pattern and top-k masker bases (reference: maskers/fixed/base.py:13-152)."""
from __future__ import annotations

from abc import abstractmethod
from dataclasses import dataclass
from typing import Any, Dict, Optional, Union

import torch

from ....utils.mask import Mask
from ....utils.native_rows import NativeRows
from ..... import _native as N
from ..base import AttentionTensorDimensions, MaskerConfig, ResearchMasker


@dataclass
class FixedMaskerConfig(MaskerConfig):
    """Base configuration for fixed pattern maskers."""


class FixedMasker(ResearchMasker):
    def __init__(self, config: FixedMaskerConfig) -> None:
        super().__init__(config)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "FixedMasker":
        if not isinstance(config, FixedMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)


@dataclass
class TopKMaskerConfig(FixedMaskerConfig):
    heavy_size: Union[float, int]

    def __post_init__(self) -> None:
        if not self.heavy_size > 0:
            raise ValueError(f"heavy_size must be > 0, got {self.heavy_size}")


def sortable_key_of(value: float, dtype: torch.dtype) -> int:
    """Host twin of the kernels' order-preserving key transform for one scalar."""
    t = torch.tensor([value], dtype=dtype)
    if dtype == torch.float32:
        u = int(t.view(torch.int32).item()) & 0xFFFFFFFF
        if u == 0x80000000:
            u = 0
        return (~u) & 0xFFFFFFFF if u & 0x80000000 else u | 0x80000000
    u = int(t.view(torch.int16).item()) & 0xFFFF
    if u == 0x8000:
        u = 0
    return (~u) & 0xFFFF if u & 0x8000 else u | 0x8000


class TopKMasker(FixedMasker):
    """Top-k over the columns not yet active, ties to the lowest column."""

    def __init__(self, config: TopKMaskerConfig) -> None:
        super().__init__(config)

    def _get_topk_indices_from_inactive_positions(self, scores: torch.Tensor, previous_mask: Mask, k: int) -> torch.Tensor:
        """Row-wise indices of the k best inactive columns (container utility mirroring
        fixed/base.py:74-85; ties resolve to the lowest column via a stable sort)."""
        masked = scores.clone()
        masked[previous_mask.get_dense_mask() != 0] = float("-inf")
        order = torch.argsort(masked, dim=-1, descending=True, stable=True)
        return order[..., :k]

    def _select_into_rows(
        self,
        rows: NativeRows,
        keys_buf: torch.Tensor,
        key_bits: int,
        n_cand: int,
        col_offset: int,
        k: int,
        excluded_key: int,
    ) -> None:
        """sah_select_topk over sortable keys [n_rows, pitch]; extends `rows` in place."""
        rows.zero_if_fresh()
        args = N.SelectTopkArgs(
            rows.as_struct(), keys_buf.data_ptr(), keys_buf.stride(0), key_bits, n_cand, col_offset, k,
            excluded_key, 0, 0, 0, N.stream_ptr(rows.device),
        )
        N.call("sah_select_topk", args)
        # every row gains exactly k entries when it certainly has k inactive candidates left
        rows.note_added(k, exact=(n_cand - rows.max_cnt >= k))

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "TopKMasker":
        if not isinstance(config, TopKMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)


@dataclass
class TopPMaskerConfig(FixedMaskerConfig):
    top_p: float

    def __post_init__(self) -> None:
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError(f"top_p must be in range [0, 1], got {self.top_p}")
