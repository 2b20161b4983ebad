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


class AdditiveMaskFacts:
    """What the additive mask of the current forward pass holds, established once per mask tensor.

    HuggingFace builds one mask per forward pass and hands the same tensor to every layer; for a single decode
    query of an unpadded batch its eager mask is all zeros, and adding zeros to scores and logits changes nothing
    (reference: hashattention_top_k.py:367-368, oracle_top_k.py:71-72, utils/mask_attention_utils.py:221-225).
    `all_zero` asks the device once per tensor (one small launch and one read-back, over the mask's whole width: a
    mask that is zero everywhere is zero on the columns of any key count) and remembers the answer for as long as
    the same, unmodified tensor keeps arriving; the tensor is kept referenced meanwhile, so its memory cannot be
    handed to another tensor that would then be mistaken for it."""

    def __init__(self) -> None:
        self._tensor: Optional[torch.Tensor] = None
        self._version = -1
        self._flags = 0

    def flags(self, attention_mask: torch.Tensor) -> int:
        am = attention_mask
        if am is self._tensor and am._version == self._version:
            return self._flags
        if am.dim() != 4 or am.stride(-1) != 1 or not am.is_cuda or am.numel() == 0:
            return N.AMASK_NONZERO | N.AMASK_GENERAL  # nothing established: every consumer reads the mask itself
        out = torch.zeros(1, dtype=torch.int32, device=am.device)
        N.call("sah_amask_classify", N.AmaskClassifyArgs(
            am.data_ptr(), am.stride(0), am.stride(1), am.stride(2), N.dtype_code(am.dtype),
            am.shape[0], am.shape[1], am.shape[2], am.shape[3], out.data_ptr(), N.stream_ptr(am.device)))
        self._flags = int(out.item())
        self._tensor, self._version = am, am._version
        return self._flags

    def all_zero(self, attention_mask: torch.Tensor) -> bool:
        return self.flags(attention_mask) == 0


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
    return_stats: bool = False,
    dropout: Tuple[float, int, int] = (0.0, 0, 0),
    dropout_numerator_only: bool = False,
    score_keys: Optional[Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """rows=None => dense attention over all keys. `return_stats`: the second value is the kernel's
    fp32 (n_rows, 2) tensor of (largest logit among the row's entries, softmax denominator relative to it)
    instead of the dense probabilities. `score_keys`: the (n_rows, >= Lk) 16-bit keys and remainders
    `sah_qk_scores` wrote for these queries and keys without an additive mask, when a masker of this call has scored
    every key already - the kernel then takes its logits from there and does not read K."""
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
    if return_attention_weights or return_stats:
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
        dropout[0], dropout[1], dropout[2], int(dropout_numerator_only),
    )
    sk, sr = score_keys if score_keys is not None else (None, None)
    if (sk is not None and sr is not None and not dense and sk.dtype == torch.int16 and sk.device == dev
            and sk.ndim == 2 and sk.shape[0] == n_rows and sk.stride(1) == 1 and sk.stride(0) >= Lk
            and sr.dtype == sk.dtype and sr.shape == sk.shape and sr.stride() == sk.stride()):
        args.score_keys, args.score_resid, args.score_pitch = sk.data_ptr(), sr.data_ptr(), sk.stride(0)
    N.call("sah_sparse_attention", args)
    if return_stats:
        return out, stats
    weights = None
    if return_attention_weights:
        weights = torch.zeros((B, Hq, Lq, Lk), dtype=q.dtype, device=dev)
        wargs = N.AttentionWeightsArgs(
            rows_struct, logits.data_ptr(), stats.data_ptr(), unit, 1 if dense else 0, dt,
            weights.data_ptr(), N.stream_ptr(dev), dropout[0], dropout[1], dropout[2],
        )
        N.call("sah_attention_weights", wargs)
    return out, weights


def _training_dropout(module: Optional[nn.Module], dropout: float) -> Tuple[float, int, int]:
    """(p, seed, offset) for the attention kernel: dropout of the exp weights applies in training mode only
    (reference: mask_attention_utils.py:234-238, `module.training`). The kernel draws with Philox4x32-10 keyed by
    torch's seed and a per-call offset where the reference draws from torch's generator: another stream of the same
    distribution. The offset is itself a draw from torch's default generator, so `torch.manual_seed(s)` followed by the
    same calls gives the same dropout masks again, as it does in the reference."""
    if not (dropout > 0.0 and module is not None and getattr(module, "training", False)):
        return 0.0, 0, 0
    if not dropout < 1.0:
        raise ValueError(f"dropout probability has to be below 1 for the attention kernel, but got {dropout}")
    offset = int(torch.randint(0, 2 ** 62, (1,), dtype=torch.int64).item())
    return float(dropout), int(torch.initial_seed()) & 0xFFFFFFFFFFFFFFFF, offset


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
    """Dense attention output (B, Lq, Hq, D) (reference: mask_attention_utils.py:11-70). In training mode the
    reference's dense path is scaled_dot_product_attention with dropout_p (:40-52): dropout of the normalised
    probabilities, i.e. a dropped entry leaves the softmax denominator as it is."""
    out, _ = _run_attention(queries, keys, values, attention_mask, None, scaling, None, False,
                            dropout=_training_dropout(module, dropout), dropout_numerator_only=True)
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
    mask = sparse_attention_mask
    if mask.is_full or mask.is_empty:
        rows = None
    else:
        rows = mask.to_rows(0)
    out, weights = _run_attention(
        queries, keys, values, attention_mask, sinks, scaling, rows, return_attention_weights,
        dropout=_training_dropout(module, dropout), score_keys=kwargs.get("_score_keys"),
    )
    if return_attention_weights:
        return out, weights
    return out


# ------------------------------------------------------------------ numerator / denominator helpers
def _masked_softmax_parts(queries, keys, values, attention_mask, scaling, mask: Mask, dropout=(0.0, 0, 0)):
    """(out (B, Hq, Lq, D) fp32, den (B, Hq, Lq, 1) fp32, m_all (B, Hq, Lq, 1) fp32) of the masked softmax in the
    reference's scale, i.e. relative to the largest logit over ALL keys of the row
    (mask_attention_utils.py:187-240). Two launches of the attention kernel: one over the mask's rows, one dense
    pass whose statistics give the all-key maximum."""
    B, Hq, Lq, D = queries.shape
    rows = None if (mask.is_full or mask.is_empty) else mask.to_rows(0)
    out, stats = _run_attention(queries, keys, values, attention_mask, None, scaling, rows, False, return_stats=True,
                                dropout=dropout)
    if rows is None:
        all_stats = stats
    else:
        _, all_stats = _run_attention(queries, keys, values, attention_mask, None, scaling, None, False, return_stats=True)
    m_sel = stats[:, 0].view(B, Hq, Lq, 1)
    m_all = all_stats[:, 0].view(B, Hq, Lq, 1)
    den = stats[:, 1].view(B, Hq, Lq, 1) * torch.exp(m_sel - m_all)
    return out.transpose(1, 2).to(torch.float32), den, m_all


def get_attention_denominator(module: Optional[nn.Module], queries: torch.Tensor, keys: torch.Tensor,
                              attention_mask: Optional[torch.Tensor], scaling: float, dropout: float,
                              sparse_attention_mask: Mask, **kwargs: Dict[str, Any]) -> torch.Tensor:
    """sum_j exp(z_j - max_all z) / (w_j + 1e-6) over the mask's entries, (B, Hq, Lq, 1) fp32
    (reference: mask_attention_utils.py:271-311). The kernel needs a value tensor: the keys stand in."""
    _, den, _ = _masked_softmax_parts(queries, keys, keys, attention_mask, scaling, sparse_attention_mask,
                                      _training_dropout(module, dropout))
    return den


def get_attention_numerator(module: Optional[nn.Module], queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor,
                            attention_mask: Optional[torch.Tensor], scaling: float, dropout: float,
                            sparse_attention_mask: Mask, **kwargs: Dict[str, Any]) -> torch.Tensor:
    """sum_j exp(z_j - max_all z) / (w_j + 1e-6) * V_j, (B, Hq, Lq, D) fp32 (reference :314-355). Rebuilt as the
    kernel's normalised output times the denominator, so for bf16 / fp16 inputs it carries the output's rounding
    (one part in 2^8 / 2^11) where the reference's fp32 product does not."""
    out, den, _ = _masked_softmax_parts(queries, keys, values, attention_mask, scaling, sparse_attention_mask,
                                        _training_dropout(module, dropout))
    return out * den


def apply_sink_bias(num: torch.Tensor, den: torch.Tensor, exp_attention_weights: Optional[torch.Tensor],
                    queries: torch.Tensor, keys: torch.Tensor, attention_mask: Optional[torch.Tensor],
                    sinks: Optional[torch.Tensor], scaling: float):
    """Adds one attention-sink logit per query head to a softmax given as (numerator, denominator[, exp weights])
    in the all-key-maximum scale: everything is rescaled by exp(old_max - max(old_max, sink)) and the
    denominator gains exp(sink - new_max) (reference :357-402). The all-key maximum comes from a dense pass of
    the attention kernel; the rest is arithmetic on (B, Hq, Lq, 1) tensors."""
    if sinks is None:
        return num, den, exp_attention_weights
    assert sinks.ndim == 1, f"sinks must be 1D tensor of shape [H], got {sinks.shape}"
    B, H, Q = queries.shape[0], queries.shape[1], queries.shape[2]
    _, stats = _run_attention(queries, keys, keys, attention_mask, None, scaling, None, False, return_stats=True)
    old_max = stats[:, 0].view(B, H, Q, 1)
    sinks_row = sinks.to(device=old_max.device, dtype=torch.float32).view(1, H, 1, 1).expand(B, H, Q, 1)
    new_max = torch.maximum(old_max, sinks_row)
    scale = torch.exp(old_max - new_max).to(den.dtype)
    num = num * scale
    den = den * scale
    if exp_attention_weights is not None:
        exp_attention_weights = exp_attention_weights * scale
    den = den + torch.exp(sinks_row - new_max).to(den.dtype)
    return num, den, exp_attention_weights


def create_sampling_mask_with_per_head_budget(budgets: torch.Tensor, sampling_probability: torch.Tensor,
                                              seq_len_keys: int, start_idx: int, end_idx: int,
                                              dtype: torch.dtype = torch.float32, seed: Optional[int] = None,
                                              offset: int = 0) -> Mask:
    """Mask (B, H, Lq, seq_len_keys) in which row r holds the DISTINCT columns among `budgets[r]` uniform draws
    (with replacement) from [start_idx, end_idx), each with weight `sampling_probability[r]` rounded to `dtype`
    (reference: mask_attention_utils.py:105-184, one `sah_adaptive_sample` launch here, no host
    synchronisation). The reference lists a column once per draw in its index form; every consumer
    (dense conversion, merge) collapses such repeats to the one weight, which is what the rows hold here.
    Draws are Philox4x32-10 with key `seed` (default torch.initial_seed()) and stream `offset`."""
    if budgets.dim() != 4 or budgets.shape[-1] != 1 or sampling_probability.shape != budgets.shape:
        raise ValueError(f"budgets and sampling_probability must both be (b, h, q, 1), got {tuple(budgets.shape)} "
                         f"and {tuple(sampling_probability.shape)}")
    N.require_device(budgets, "budgets")
    B, H, Lq, _ = budgets.shape
    n = int(end_idx) - int(start_idx)
    if n <= 0 or start_idx < 0 or end_idx > seq_len_keys:
        raise ValueError(f"sampling range [{start_idx}, {end_idx}) is outside the {seq_len_keys} keys")
    dev = budgets.device
    n_rows = B * H * Lq
    rows = NativeRows(n_rows, int(seq_len_keys), n, dev, weighted=True)
    rows.zero_if_fresh()
    bud = budgets.reshape(n_rows).to(torch.int32).contiguous()
    N.dtype_code(dtype)
    prob = sampling_probability.reshape(n_rows).to(dtype).to(torch.float32).contiguous()
    key = (torch.initial_seed() if seed is None else int(seed)) & 0xFFFFFFFFFFFFFFFF
    N.call("sah_adaptive_sample", N.AdaptiveSampleArgs(
        rows.as_struct(), bud.data_ptr(), prob.data_ptr(), N.dtype_code(dtype),
        int(start_idx), n, key, int(offset), 1, N.stream_ptr(dev),
    ))
    rows.note_added(n, exact=False)
    return Mask.create_mask_from_rows((B, H, Lq, int(seq_len_keys)), rows, dtype)
