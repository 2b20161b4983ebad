"""Masked-softmax attention over the selected KV rows.

Host side of `sah_sparse_attention` (include/sah.h). Same call signature and
results as the reference's `get_masked_attention_output`
(sparse_attention/utils/mask_attention_utils.py:406-491), which computes
fp32 logits over *all* keys, multiplies exp(logit - rowmax) by the inverse mask
weight 1/(w + 1e-6) and divides numerator by denominator; here only the rows the
mask selects are read (an empty or full mask selects every key, as in the
reference, utils/mask.py:733-735).
"""
from __future__ import annotations

from typing import Any, Dict, Optional, Tuple, Union

import numpy as np
import torch
from torch import nn

from ... import _native as N
from .kv_utils import _get_num_key_value_groups
from .mask import Mask
from .native_rows import NativeRows

_WORK: Dict[Tuple[str, int], torch.Tensor] = {}


def _workspace(device: torch.device, floats: int) -> torch.Tensor:
    """Grow-only fp32 scratch per device; reused across calls on the same stream."""
    key = (device.type, device.index if device.index is not None else -1)
    buf = _WORK.get(key)
    if buf is None or buf.numel() < floats:
        buf = torch.empty(max(floats, 1 << 16), dtype=torch.float32, device=device)
        _WORK[key] = buf
    return buf


def _inner_contiguous(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


def unit_inverse_weight(dtype: torch.dtype) -> float:
    """1 / (1 + 1e-6) evaluated in the mask dtype, as `Mask.apply_inv_mask` does for weight 1.0."""
    if dtype == torch.float32:
        return float(np.float32(1.0) / (np.float32(1.0) + np.float32(1e-6)))
    return 1.0  # bf16 / fp16: 1 + 1e-6 rounds back to 1


def additive_mask_args(attention_mask: Optional[torch.Tensor], queries: torch.Tensor, n_keys: int):
    """(tensor kept alive, ptr, stride_b, stride_h, stride_q) of the additive mask or all-None/0."""
    if attention_mask is None:
        return None, None, 0, 0, 0
    am = attention_mask
    if am.dim() != 4:
        raise ValueError(f"attention_mask must have 4 dimensions, got shape {tuple(am.shape)}")
    B, H, Lq = queries.shape[0], queries.shape[1], queries.shape[2]
    if am.shape[-1] < n_keys or am.shape[2] != Lq or am.shape[0] not in (1, B) or am.shape[1] not in (1, H):
        raise ValueError(f"attention_mask shape {tuple(am.shape)} does not cover queries {tuple(queries.shape)} x {n_keys} keys")
    if am.dtype != queries.dtype:
        am = am.to(queries.dtype)
    am = _inner_contiguous(am)
    N.require_device(am, "attention_mask")
    sb = am.stride(0) if am.shape[0] > 1 else 0
    sh = am.stride(1) if am.shape[1] > 1 else 0
    return am, am.data_ptr(), sb, sh, am.stride(2)


def _run_attention(
    queries: torch.Tensor,
    keys: torch.Tensor,
    values: torch.Tensor,
    attention_mask: Optional[torch.Tensor],
    sinks: Optional[torch.Tensor],
    scaling: float,
    rows: Optional[NativeRows],
    return_attention_weights: bool,
    out: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """rows=None => dense attention over all keys."""
    N.require_device(queries, "queries")
    N.require_device(keys, "keys")
    N.require_device(values, "values")
    B, Hq, Lq, D = queries.shape
    Hkv, Lk = keys.shape[1], keys.shape[2]
    _get_num_key_value_groups(queries, keys)
    _get_num_key_value_groups(queries, values)
    if keys.dtype != queries.dtype or values.dtype != queries.dtype:
        raise ValueError(f"queries/keys/values dtypes differ: {queries.dtype}, {keys.dtype}, {values.dtype}")
    q = _inner_contiguous(queries)
    k = _inner_contiguous(keys)
    v = _inner_contiguous(values)
    dev = q.device
    dt = N.dtype_code(q.dtype)
    n_rows = B * Hq * Lq
    dense = rows is None
    if dense:
        max_cnt = Lk
        rows_struct = N.Rows(None, None, None, None, n_rows, Lk, Lk, (Lk + 31) // 32)
        unit = 1.0
    else:
        rows.zero_if_fresh()
        max_cnt = max(1, rows.max_cnt)
        rows_struct = rows.as_struct()
        unit = unit_inverse_weight(q.dtype)
    am_keep, am_ptr, ms_b, ms_h, ms_l = additive_mask_args(attention_mask, q, Lk)
    sink_t = None
    if sinks is not None:
        assert sinks.ndim == 1, f"sinks must be 1D tensor of shape [H], got {sinks.shape}"
        sink_t = sinks.to(device=dev, dtype=torch.float32).contiguous()
    if out is None:
        out = torch.empty((B, Lq, Hq, D), dtype=q.dtype, device=dev)
    floats = N.work_floats(n_rows, max_cnt, D)
    work = _workspace(dev, floats)
    logits = stats = None
    if return_attention_weights:
        logits = torch.empty((n_rows, Lk if dense else rows.cap), dtype=torch.float32, device=dev)
        stats = torch.empty((n_rows, 2), dtype=torch.float32, device=dev)
    args = N.AttentionArgs(
        rows_struct,
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
        k.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
        v.data_ptr(), v.stride(0), v.stride(1), v.stride(2),
        am_ptr, ms_b, ms_h, ms_l,
        None if sink_t is None else sink_t.data_ptr(),
        dt, B, Hq, Hkv, Lq, Lk, D,
        float(scaling), unit,
        1 if dense else 0,
        0, 0, 0,
        max_cnt,
        out.data_ptr(),
        work.data_ptr(), work.numel(),
        None if logits is None else logits.data_ptr(),
        None if stats is None else stats.data_ptr(),
        N.stream_ptr(dev),
    )
    N.call("sah_sparse_attention", args)
    weights = None
    if return_attention_weights:
        weights = torch.zeros((B, Hq, Lq, Lk), dtype=q.dtype, device=dev)
        wargs = N.AttentionWeightsArgs(
            rows_struct, logits.data_ptr(), stats.data_ptr(), unit, 1 if dense else 0, dt,
            weights.data_ptr(), N.stream_ptr(dev),
        )
        N.call("sah_attention_weights", wargs)
    return out, weights


def _reject_training_dropout(module: Optional[nn.Module], dropout: float) -> None:
    if dropout > 0.0 and module is not None and getattr(module, "training", False):
        raise NotImplementedError(
            "attention dropout in training mode is not implemented by the MI355X decode kernels"
        )


def get_true_attention_output(
    module: nn.Module,
    queries: torch.Tensor,
    keys: torch.Tensor,
    values: torch.Tensor,
    attention_mask: Optional[torch.Tensor],
    scaling: float,
    dropout: float,
    **kwargs: Dict[str, Any],
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Dense attention output (B, Lq, Hq, D) (reference: mask_attention_utils.py:11-70)."""
    _reject_training_dropout(module, dropout)
    out, _ = _run_attention(queries, keys, values, attention_mask, None, scaling, None, False)
    return out, None


def apply_inv_mask_sum(input_tensor: torch.Tensor, mask: Mask) -> torch.Tensor:
    """sum over the last dim of mask.apply_inv_mask(x); full/empty masks sum x (reference :73-101)."""
    if tuple(input_tensor.shape) != tuple(mask.shape):
        raise ValueError(f"input_tensor.shape must be {mask.shape}, got {input_tensor.shape}")
    if mask.is_full or mask.is_empty:
        return input_tensor.sum(dim=-1, keepdim=True)
    return mask.apply_inv_mask(input_tensor).sum(dim=-1, keepdim=True)


def get_masked_attention_output(
    module: nn.Module,
    queries: torch.Tensor,
    keys: torch.Tensor,
    values: torch.Tensor,
    attention_mask: Optional[torch.Tensor],
    sinks: Optional[torch.Tensor],
    scaling: float,
    dropout: float,
    sparse_attention_mask: Mask,
    return_attention_weights: bool = False,
    **kwargs: Dict[str, Any],
) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """Masked attention output (B, Lq, Hq, D) in the query dtype, optionally with the
    dense probabilities (B, Hq, Lq, Lk)."""
    _reject_training_dropout(module, dropout)
    mask = sparse_attention_mask
    if mask.is_full or mask.is_empty:
        rows = None
    else:
        rows = mask.to_rows(0)
    out, weights = _run_attention(
        queries, keys, values, attention_mask, sinks, scaling, rows, return_attention_weights
    )
    if return_attention_weights:
        return out, weights
    return out
