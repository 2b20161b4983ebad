"""RandomSamplingMasker: a fixed fraction of uniformly drawn key positions per query row.

Reference (maskers/sampling/implementations/random_sampling.py:25-193): per row int(rate * n_keys) draws,
uniform on [0, n_keys), with replacement (so fewer distinct columns than draws); every drawn column gets the
weight `rate` and the result is merged into the previous mask by clamp(previous + rate, 0, 1). A full previous
mask is returned as it is. Here the draws and the merge are one launch of the adaptive sampler's kernel
(`sah_adaptive_sample`) with the same budget in every row; draws come from Philox4x32-10 keyed by `seed`
(default: torch.initial_seed()) and a per-call offset instead of torch's global generator.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Optional

import torch

from .....utils.mask import Mask
from ...... import _native as N
from ...base import AttentionTensorDimensions, MaskerConfig, MaskerRegistry
from ..base import SamplingMasker, SamplingMaskerConfig


@dataclass
class RandomSamplingMaskerConfig(SamplingMaskerConfig):
    sampling_rate: float
    search_space: Dict[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        if not (0.0 < self.sampling_rate <= 1.0):
            raise ValueError(f"sampling_rate must be in range (0, 1], got {self.sampling_rate}")


@MaskerRegistry.register(RandomSamplingMaskerConfig)
class RandomSamplingMasker(SamplingMasker):
    sampling_rate: float

    def __init__(self, config: RandomSamplingMaskerConfig) -> None:
        super().__init__(config)
        self.sampling_rate = config.sampling_rate
        self.seed: Optional[int] = None  # Philox key; None = torch.initial_seed() at call time
        self.call_index = 0              # call c draws with Philox offset c

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        return int(self.sampling_rate * dims.seq_len_keys)

    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        if previous_mask.is_full_mask():
            return previous_mask
        dims = self._extract_tensor_dimensions(keys, queries)
        Lk = dims.seq_len_keys
        n_draws = int(self.sampling_rate * Lk)
        if n_draws <= 0:
            return previous_mask  # merging a mask without entries changes nothing
        if Lk < 2:
            return self._create_full_mask(dims, previous_mask.dtype, previous_mask.device)
        N.require_device(queries, "queries")
        rows = previous_mask.to_rows(extra=min(n_draws, Lk))
        rows.zero_if_fresh()
        w_fresh = rows.w is None
        if w_fresh:
            rows.w = torch.empty((rows.n_rows, rows.cap), dtype=torch.float32, device=queries.device)
        budget = torch.full((rows.n_rows,), n_draws, dtype=torch.int32, device=queries.device)
        # the weight is the rate in the mask's dtype (torch.full_like(..., dtype=previous_mask.dtype), :165-170)
        rate = float(torch.tensor(self.sampling_rate, dtype=previous_mask.dtype).float())
        prob = torch.full((rows.n_rows,), rate, dtype=torch.float32, device=queries.device)
        seed = (torch.initial_seed() if self.seed is None else int(self.seed)) & 0xFFFFFFFFFFFFFFFF
        offset = self.call_index
        self.call_index += 1
        N.call("sah_adaptive_sample", N.AdaptiveSampleArgs(
            rows.as_struct(), budget.data_ptr(), prob.data_ptr(), N.dtype_code(previous_mask.dtype),
            0, Lk, seed, offset, int(w_fresh), N.stream_ptr(queries.device),
        ))
        rows.note_added(min(n_draws, Lk), exact=False)
        return Mask.create_mask_from_rows(self._mask_shape(dims), rows, previous_mask.dtype)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "RandomSamplingMasker":
        if not isinstance(config, RandomSamplingMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)
