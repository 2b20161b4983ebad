"""Sink and Local maskers on the fused index builder `sah_sink_local_indices`.

Reference behaviour (maskers/fixed/implementations/basic_fixed.py):
  * SinkMasker  (:311-462): columns [0, sink) of every row; Lk <= sink -> full mask.
  * LocalMasker (:18-276):  for query row q the columns [Lk-Lq-w+1+q, Lk-Lq+q];
    Lk <= w + Lq -> full mask; columns beyond Lk-Lq+q are cleared, including ones
    an earlier masker set (:60-66).
  * CausalMasker (:279-308): returns the previous mask unchanged.
The reference fills a dense (B,Hq,Lq,Lk) tensor; here the column list, the
per-row count and the membership bitmap are written directly.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Optional, Union

import torch

from .....utils.mask import Mask
from ...... import _native as N
from ...base import AttentionTensorDimensions, MaskerConfig, MaskerRegistry
from ..base import FixedMasker, FixedMaskerConfig


def _launch_sink_local(rows, lq: int, sink: int, window: int, clear_future: bool) -> None:
    fresh = rows.fresh
    args = N.SinkLocalArgs(rows.as_struct(), lq, sink, window, 1 if fresh else 0, 1 if clear_future else 0,
                           N.stream_ptr(rows.device))
    N.call("sah_sink_local_indices", args)
    added = min(sink, rows.n_keys) + window
    # exact when the rows were empty and the two ranges cannot overlap for any query row
    exact = fresh and (window == 0 or sink == 0 or rows.n_keys - lq - window + 1 >= sink) and lq == 1
    rows.note_added(added, exact=exact)


@dataclass
class LocalMaskerConfig(FixedMaskerConfig):
    window_size: Union[float, int]
    search_space: Dict[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        if not self.window_size > 0:
            raise ValueError(f"window_size must be > 0, got {self.window_size}")


@MaskerRegistry.register(LocalMaskerConfig)
class LocalMasker(FixedMasker):
    window_size: Union[float, int]

    def __init__(self, config: LocalMaskerConfig) -> None:
        super().__init__(config)
        self.window_size = config.window_size

    def _calculate_effective_window_size(self, seq_len_keys: int) -> int:
        return self._calculate_effective_size(self.window_size, seq_len_keys)

    def _should_use_full_attention(self, dims: AttentionTensorDimensions, window_size: int) -> bool:
        return dims.seq_len_keys <= window_size + dims.seq_len_queries

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        return self._calculate_effective_window_size(dims.seq_len_keys)

    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        if previous_mask.is_full_mask():
            return previous_mask
        dims = self._extract_tensor_dimensions(keys, queries)
        window = self._calculate_effective_window_size(dims.seq_len_keys)
        if self._should_use_full_attention(dims, window):
            return self._create_full_mask(dims, previous_mask.dtype, previous_mask.device)
        N.require_device(keys, "keys")
        rows = previous_mask.to_rows(extra=window)
        _launch_sink_local(rows, dims.seq_len_queries, 0, window, clear_future=True)
        return Mask.create_mask_from_rows(self._mask_shape(dims), rows, previous_mask.dtype)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "LocalMasker":
        if not isinstance(config, LocalMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)


@MaskerRegistry.register(FixedMaskerConfig)
class CausalMasker(FixedMasker):
    """Placeholder of the reference: hands the previous mask back."""

    def __init__(self, config: FixedMaskerConfig) -> None:
        super().__init__(config)

    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        return previous_mask

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "CausalMasker":
        if not isinstance(config, FixedMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)


@dataclass
class SinkMaskerConfig(FixedMaskerConfig):
    sink_size: Union[float, int]
    search_space: Dict[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        if not self.sink_size > 0:
            raise ValueError(f"sink_size must be > 0, got {self.sink_size}")


@MaskerRegistry.register(SinkMaskerConfig)
class SinkMasker(FixedMasker):
    sink_size: Union[float, int]

    def __init__(self, config: SinkMaskerConfig) -> None:
        super().__init__(config)
        self.sink_size = config.sink_size

    def _calculate_effective_sink_size(self, seq_len_keys: int) -> int:
        return self._calculate_effective_size(self.sink_size, seq_len_keys)

    def _should_use_full_attention(self, dims: AttentionTensorDimensions, sink_size: int) -> bool:
        return dims.seq_len_keys <= sink_size

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        return self._calculate_effective_sink_size(dims.seq_len_keys)

    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        if previous_mask.is_full_mask():
            return previous_mask
        dims = self._extract_tensor_dimensions(keys, queries)
        sink = self._calculate_effective_sink_size(dims.seq_len_keys)
        if self._should_use_full_attention(dims, sink):
            return self._create_full_mask(dims, previous_mask.dtype, previous_mask.device)
        N.require_device(keys, "keys")
        if sink <= 0:
            return previous_mask
        rows = previous_mask.to_rows(extra=sink)
        _launch_sink_local(rows, dims.seq_len_queries, sink, 0, clear_future=False)
        return Mask.create_mask_from_rows(self._mask_shape(dims), rows, previous_mask.dtype)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "SinkMasker":
        if not isinstance(config, SinkMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)


def fused_sink_local(sink_masker: SinkMasker, local_masker: LocalMasker, keys: torch.Tensor, queries: torch.Tensor,
                     previous_mask: Mask) -> Mask:
    """SinkMasker.add_mask followed by LocalMasker.add_mask on an empty previous mask, as one
    `sah_sink_local_indices` launch. Same results as the two calls, including the full-mask
    short-circuits of either masker."""
    if not previous_mask.is_empty_mask():
        raise ValueError("fused_sink_local needs an empty previous mask")
    dims = sink_masker._extract_tensor_dimensions(keys, queries)
    sink = sink_masker._calculate_effective_sink_size(dims.seq_len_keys)
    window = local_masker._calculate_effective_window_size(dims.seq_len_keys)
    if sink_masker._should_use_full_attention(dims, sink) or local_masker._should_use_full_attention(dims, window):
        return sink_masker._create_full_mask(dims, previous_mask.dtype, previous_mask.device)
    N.require_device(keys, "keys")
    rows = previous_mask.to_rows(extra=max(0, sink) + window)
    if not rows.fresh:
        raise ValueError("fused_sink_local needs uninitialised rows")
    _launch_sink_local(rows, dims.seq_len_queries, max(0, sink), window, clear_future=True)
    return Mask.create_mask_from_rows(sink_masker._mask_shape(dims), rows, previous_mask.dtype)
