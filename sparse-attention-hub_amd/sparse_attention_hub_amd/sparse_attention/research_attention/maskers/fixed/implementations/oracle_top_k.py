"""OracleTopK: exact QK scores, top-k of the not-yet-active keys.

Reference (maskers/fixed/implementations/oracle_top_k.py:48-125): scores =
matmul(queries, repeat_kv(keys)^T), un-scaled and in the query dtype, plus the
additive attention mask; already-active columns are set to finfo(dtype).min;
torch.topk picks k columns which are then set to 1.0. Here one pass over K per KV
head (`sah_qk_scores`) serves the whole GQA group and `sah_select_topk` does the
selection with the lowest-column tie rule, appending straight to the row lists.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Optional, Union

import torch

from .....utils.kv_utils import _get_num_key_value_groups
from .....utils.mask import Mask
from .....utils.mask_attention_utils import _inner_contiguous, additive_mask_args
from ...... import _native as N
from ...base import AttentionTensorDimensions, MaskerConfig, MaskerRegistry
from ..base import TopKMasker, TopKMaskerConfig, sortable_key_of

_HEAVY_GRID = [0.01, 0.02, 0.03, 0.04, 0.05, 0.06, 0.07, 0.08, 0.09, 0.1]


def _default_search_space() -> Dict[str, Any]:
    """The reference's Ray Tune grid when ray is installed, the plain list otherwise."""
    try:
        from ray import tune  # type: ignore

        return {"heavy_size": tune.grid_search(list(_HEAVY_GRID))}
    except Exception:
        return {"heavy_size": list(_HEAVY_GRID)}


@dataclass
class OracleTopKConfig(TopKMaskerConfig):
    search_space: Dict[str, Any] = field(default_factory=_default_search_space)


def score_key_buffer(n_rows: int, n_cols: int, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """Scratch for sortable keys: 16-bit for bf16/fp16 scores, 32-bit for fp32."""
    kdt = torch.int32 if dtype == torch.float32 else torch.int16
    pitch = (n_cols + 63) // 64 * 64
    return torch.empty((n_rows, pitch), dtype=kdt, device=device)


def score_remainder_buffer(keybuf: torch.Tensor, head_dim: int, masked: bool) -> Optional[torch.Tensor]:
    """Beside 16-bit score keys of an unmasked scoring pass: room for what the scores' rounding took away
    (`sah_qk_scores_args.resid_out`), with which the attention of the same call need not read K again. None where the
    kernels have no use for it (fp32 tensors, an additive mask in the scores, head_dim other than 64 / 128)."""
    if masked or keybuf.dtype != torch.int16 or head_dim not in (64, 128):
        return None
    return torch.empty_like(keybuf)


@MaskerRegistry.register(OracleTopKConfig)
class OracleTopK(TopKMasker):
    heavy_size: Union[float, int]

    def __init__(self, config: OracleTopKConfig) -> None:
        super().__init__(config)
        self.heavy_size = config.heavy_size

    def _calculate_effective_heavy_size(self, seq_len_keys: int) -> int:
        return self._calculate_effective_size(self.heavy_size, seq_len_keys)

    def _should_use_full_attention(self, dims: AttentionTensorDimensions, heavy_size: int) -> bool:
        return dims.seq_len_keys <= heavy_size

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        return self._calculate_effective_heavy_size(dims.seq_len_keys)

    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        if previous_mask.is_full_mask():
            return previous_mask
        dims = self._extract_tensor_dimensions(keys, queries)
        k_eff = self._calculate_effective_heavy_size(dims.seq_len_keys)
        if self._should_use_full_attention(dims, k_eff):
            return self._create_full_mask(dims, previous_mask.dtype, previous_mask.device)
        if k_eff <= 0:
            return previous_mask
        N.require_device(keys, "keys")
        N.require_device(queries, "queries")
        _get_num_key_value_groups(queries, keys)
        B, Hq, Lq, D = queries.shape
        Hkv, Lk = keys.shape[1], keys.shape[2]
        q = _inner_contiguous(queries)
        k = _inner_contiguous(keys)
        rows = previous_mask.to_rows(extra=k_eff)
        keybuf = score_key_buffer(rows.n_rows, Lk, q.dtype, q.device)
        am_keep, am_ptr, ms_b, ms_h, ms_l = additive_mask_args(attention_mask, q, Lk)
        shared = kwargs.get("_call_scratch")
        resid = score_remainder_buffer(keybuf, D, am_ptr is not None) if isinstance(shared, dict) else None
        args = N.QkScoresArgs(
            q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
            k.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
            am_ptr, ms_b, ms_h, ms_l,
            N.dtype_code(q.dtype), B, Hq, Hkv, Lq, Lk, D,
            keybuf.data_ptr(), keybuf.stride(0), N.stream_ptr(q.device),
            None if resid is None else resid.data_ptr(),
        )
        N.call("sah_qk_scores", args)
        if am_ptr is None and isinstance(shared, dict):
            shared["qk_score_keys"] = keybuf  # later maskers of this call can skip their own scoring pass
            shared["qk_score_resid"] = resid  # ... and the attention its reading of K
            # ... and know that the largest key of every row now belongs to a column of the row: the k_eff >= 1
            # largest keys outside the previous mask were just added
            shared["qk_top_in_rows"] = True
        # active columns rank where `scores[prev != 0] = finfo(mask dtype).min` puts them
        excluded = sortable_key_of(torch.finfo(previous_mask.dtype).min, q.dtype)
        self._select_into_rows(rows, keybuf, 32 if q.dtype == torch.float32 else 16, Lk, 0, k_eff, excluded)
        return Mask.create_mask_from_rows(self._mask_shape(dims), rows, previous_mask.dtype)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "OracleTopK":
        if not isinstance(config, OracleTopKConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)
