"""AdaptiveSamplingMasker (vAttention): base sample -> per-row budget -> uniform sample.

Reference (maskers/sampling/implementations/adaptive_sampling.py:35-424): per mask row,
  e[j]   = exp(q.k_j * scaling + attention_mask - rowmax) in the query dtype, over ALL keys;
  static = sum of e over the previous mask's entries, each times 1/(w + 1e-6)
           (plain sum over all keys when the previous mask is empty);
  base   = max(2, int(rate * n)) uniform draws with replacement on [start, end), n = end - start;
  sigma  = unbiased std of e over the draws; estimate = static + sum over the distinct drawn
           columns of e / (base/n + 1e-6);
  budget = clamp(((ppf(1-delta) * sigma * n) / max(epsilon * estimate, 1e-8))^2, 1, n), at
           least `base`; p = budget / n;
  `budget` fresh uniform draws; the distinct drawn columns are merged into the previous mask
  with weight p (clamp(previous + p, 0, 1)).
The reference materialises the dense numerators and a dense sampling mask, and synchronises
once to size its index tensor. Here the numerators are recomputed inside two kernels from the
2-byte order-preserving score keys of the QK scoring pass (shared with OracleTopK when it ran in
the same call), rows grow in place with worst-case capacity, and nothing synchronises.

Random draws come from Philox4x32-10 keyed by `seed` (default: torch.initial_seed()) with a
per-call offset, not from torch's global generator: same distribution, different stream.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from statistics import NormalDist
from typing import Any, Dict, Optional, Tuple, Union

import torch

from .....utils.kv_utils import _get_num_key_value_groups
from .....utils.mask import Mask
from .....utils.mask_attention_utils import _inner_contiguous, additive_mask_args
from ...... import _native as N
from ...base import AttentionTensorDimensions, MaskerConfig, MaskerRegistry
from ...fixed.implementations.oracle_top_k import score_key_buffer, score_remainder_buffer
from ..base import SamplingMasker, SamplingMaskerConfig

_RATE_GRID = [0.01, 0.02, 0.03]
_BOUND_GRID = [0.05, 0.1, 0.2, 0.3]


def _default_search_space() -> Dict[str, Any]:
    """The reference's Ray Tune grid (adaptive_sampling.py:62-68) when ray is installed, plain lists otherwise."""
    try:
        from ray import tune  # type: ignore

        return {
            "base_rate_sampling": tune.grid_search(list(_RATE_GRID)),
            "epsilon": tune.grid_search(list(_BOUND_GRID)),
            "delta": tune.grid_search(list(_BOUND_GRID)),
        }
    except Exception:
        return {"base_rate_sampling": list(_RATE_GRID), "epsilon": list(_BOUND_GRID), "delta": list(_BOUND_GRID)}


def _check_offset(name: str, value: Union[int, float]) -> None:
    if isinstance(value, float):
        if not (0.0 <= value <= 1.0):
            raise ValueError(f"{name} must be in [0, 1] if float, got {value}")
    elif isinstance(value, int):
        if value < 0:
            raise ValueError(f"{name} must be non-negative if int, got {value}")
    else:
        raise ValueError(f"{name} must be int or float, got {type(value)}")


@dataclass
class AdaptiveSamplingMaskerConfig(SamplingMaskerConfig):
    """Fields and validation of the reference's config (adaptive_sampling.py:35-120)."""

    base_rate_sampling: Union[int, float]
    epsilon: float
    delta: float
    init_offset: Union[int, float]
    local_offset: Union[int, float]
    search_space: Dict[str, Any] = field(default_factory=_default_search_space)

    def __post_init__(self) -> None:
        rate = self.base_rate_sampling
        if isinstance(rate, float):
            if not (0.0 <= rate < 1.0):
                raise ValueError(f"base_rate_sampling must be in [0, 1) if float, got {rate}")
        elif isinstance(rate, int):
            if rate < 0:
                raise ValueError(f"base_rate_sampling must be non-negative if int, got {rate}")
        else:
            raise ValueError(f"base_rate_sampling must be int or float, got {type(rate)}")
        if not (0.0 < self.epsilon < 1.0):
            raise ValueError(f"epsilon must be in (0, 1), got {self.epsilon}")
        if not (0.0 < self.delta < 1.0):
            raise ValueError(f"delta must be in (0, 1), got {self.delta}")
        _check_offset("init_offset", self.init_offset)
        _check_offset("local_offset", self.local_offset)


@MaskerRegistry.register(AdaptiveSamplingMaskerConfig)
class AdaptiveSamplingMasker(SamplingMasker):
    base_rate_sampling: Union[int, float]
    epsilon: float
    delta: float
    init_offset: Union[int, float]
    local_offset: Union[int, float]

    def __init__(self, config: AdaptiveSamplingMaskerConfig) -> None:
        super().__init__(config)
        self.base_rate_sampling = config.base_rate_sampling
        self.epsilon = config.epsilon
        self.delta = config.delta
        self.init_offset = config.init_offset
        self.local_offset = config.local_offset
        # scipy.stats.norm.ppf(1 - delta) in the reference (:181); the standard library has the same function
        self.delta_ppf = float(NormalDist().inv_cdf(1 - self.delta))
        # Philox key; None = torch.initial_seed() at call time, so torch.manual_seed() reseeds the sampler
        self.seed: Optional[int] = None
        # number of add_mask calls that drew samples; call c uses Philox offsets 2c (base) and 2c + 1
        self.call_index = 0
        # per-row results of the last call (device tensors, never read back here)
        self.last_budget: Optional[torch.Tensor] = None
        self.last_probability: Optional[torch.Tensor] = None
        self.last_stats: Optional[torch.Tensor] = None
        self.last_rows = None
        self.keep_stats = False

    # -- reference helpers ------------------------------------------------------------------
    def should_return_full_mask(self, sampling_range: int) -> bool:
        return sampling_range < 2

    def _get_sampling_range(self, seq_len_keys: int) -> Tuple[int, int, int]:
        """(start, end, end - start) — adaptive_sampling.py:203-228; floats are fractions of the key count."""
        start = int(self.init_offset * seq_len_keys) if isinstance(self.init_offset, float) else self.init_offset
        if isinstance(self.local_offset, float):
            end = seq_len_keys - int(self.local_offset * seq_len_keys)
        else:
            end = seq_len_keys - self.local_offset
        return start, end, end - start

    def _get_base_sample_count(self, sampling_range: int) -> int:
        """At least 2 draws, since they feed a standard deviation — adaptive_sampling.py:230-235."""
        if isinstance(self.base_rate_sampling, int):
            return max(2, self.base_rate_sampling)
        return max(2, int(self.base_rate_sampling * sampling_range))

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        if self.base_rate_sampling == 0:
            return 0
        _, _, n = self._get_sampling_range(dims.seq_len_keys)
        return max(0, n)

    # -- the masker -----------------------------------------------------------------------------
    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        if previous_mask.is_full_mask():
            return previous_mask
        if self.base_rate_sampling == 0:
            return previous_mask
        dims = self._extract_tensor_dimensions(keys, queries)
        Lk = dims.seq_len_keys
        start, end, n = self._get_sampling_range(Lk)
        if self.should_return_full_mask(n):
            return self._create_full_mask(dims, previous_mask.dtype, previous_mask.device)
        if start < 0 or end > Lk:
            raise ValueError(f"sampling range [{start}, {end}) is outside the {Lk} keys")
        N.require_device(keys, "keys")
        N.require_device(queries, "queries")
        _get_num_key_value_groups(queries, keys)
        B, Hq, Lq, D = queries.shape
        Hkv = keys.shape[1]
        q = _inner_contiguous(queries)
        n_rows = B * Hq * Lq

        # score keys of round(q.k), without the additive mask: reuse the scoring pass of a
        # masker that ran earlier in this call (OracleTopK) when there is one
        shared = kwargs.get("_call_scratch")
        keybuf = shared.get("qk_score_keys") if isinstance(shared, dict) else None
        # an exact top-k over these keys ran earlier in this call: the row maximum is among the rows' entries
        max_in_rows = keybuf is not None and bool(shared.get("qk_top_in_rows"))
        if keybuf is None:
            k = _inner_contiguous(keys)
            keybuf = score_key_buffer(n_rows, Lk, q.dtype, q.device)
            resid = score_remainder_buffer(keybuf, D, False) if isinstance(shared, dict) else None
            args = N.QkScoresArgs(
                q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
                k.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
                None, 0, 0, 0,
                N.dtype_code(q.dtype), B, Hq, Hkv, Lq, Lk, D,
                keybuf.data_ptr(), keybuf.stride(0), N.stream_ptr(q.device),
                None if resid is None else resid.data_ptr(),
            )
            N.call("sah_qk_scores", args)
            if isinstance(shared, dict):
                shared["qk_score_keys"] = keybuf
                shared["qk_score_resid"] = resid

        nb = self._get_base_sample_count(n)
        prev_empty = previous_mask.is_empty_mask()
        rows = previous_mask.to_rows(extra=n)
        rows.zero_if_fresh()
        w_fresh = rows.w is None
        budget = torch.empty((n_rows,), dtype=torch.int32, device=q.device)
        prob = torch.empty((n_rows,), dtype=torch.float32, device=q.device)
        stats = torch.empty((n_rows, 4), dtype=torch.float32, device=q.device) if self.keep_stats else None
        am_keep, am_ptr, ms_b, ms_h, ms_l = additive_mask_args(attention_mask, q, Lk)
        seed = (torch.initial_seed() if self.seed is None else int(self.seed)) & 0xFFFFFFFFFFFFFFFF
        offset = 2 * self.call_index
        self.call_index += 1
        stream = N.stream_ptr(q.device)
        mask_code = N.dtype_code(previous_mask.dtype)

        N.call("sah_adaptive_budget", N.AdaptiveBudgetArgs(
            rows.as_struct(), keybuf.data_ptr(), keybuf.stride(0),
            am_ptr, ms_b, ms_h, ms_l,
            N.dtype_code(q.dtype), Hq, Lq, float(scaling),
            start, n, nb, float(self.epsilon), self.delta_ppf,
            seed, offset, int(prev_empty),
            budget.data_ptr(), prob.data_ptr(), None if stats is None else stats.data_ptr(), stream,
            int(max_in_rows and not prev_empty and am_ptr is None),
        ))
        if w_fresh:
            rows.w = torch.empty((rows.n_rows, rows.cap), dtype=torch.float32, device=q.device)
        N.call("sah_adaptive_sample", N.AdaptiveSampleArgs(
            rows.as_struct(), budget.data_ptr(), prob.data_ptr(), mask_code,
            start, n, seed, offset + 1, int(w_fresh), stream,
        ))
        rows.note_added(n, exact=False)
        self.last_budget, self.last_probability, self.last_stats, self.last_rows = budget, prob, stats, rows
        return Mask.create_mask_from_rows(self._mask_shape(dims), rows, previous_mask.dtype)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "AdaptiveSamplingMasker":
        if not isinstance(config, AdaptiveSamplingMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)
