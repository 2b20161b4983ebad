"""ResearchAttention: masker chain, then masked-softmax attention.

Reference: research_attention/base.py:24-196. Per call it starts from an empty
Mask of shape (B, Hq, Lq, Lk), lets every masker add to it in order, and hands the
result to `get_masked_attention_output`. The maskers here keep the mask in the
kernels' row layout, so one decode layer-step is a handful of HIP launches and no
dense (B, Hq, Lq, Lk) tensor unless the caller asks for the attention weights.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

import torch
from torch import nn

from ... import _native
from ...metric_logging import MicroMetricLogger
from ..base import SparseAttention, SparseAttentionConfig
from ..utils.mask import Mask
from ..utils.mask_attention_utils import AdditiveMaskFacts, get_masked_attention_output, get_true_attention_output
from ..utils.native_rows import NativeRows
from .decode_plan import DecodePlan, plan_kind
from .maskers.base import MaskerConfig, ResearchMasker
from .maskers.fixed.implementations.basic_fixed import LocalMasker, SinkMasker, fused_sink_local
from .maskers.sampling.base import SamplingMasker


# the two metrics of the reference (research_attention/base.py:20-21)
MicroMetricLogger.register_metric("research_attention_density", float)
MicroMetricLogger.register_metric("research_attention_output_error", float)


@dataclass
class ResearchAttentionConfig(SparseAttentionConfig):
    masker_configs: List[MaskerConfig]


class ResearchAttention(SparseAttention):
    maskers: List[ResearchMasker]

    # The reference always materialises the dense (B, Hq, Lq, Lk) probabilities as the
    # second return value (research_attention/base.py:146). HuggingFace attention modules
    # drop them unless output_attentions is set, so a caller may switch them off and get
    # None instead.
    return_attention_weights: bool = True

    def __init__(self, sparse_attention_config: SparseAttentionConfig, maskers: List[ResearchMasker]) -> None:
        super().__init__(sparse_attention_config)
        if sum(1 for m in maskers if isinstance(m, SamplingMasker)) > 1:
            raise ValueError(
                "Only one sampling masker supported for efficiency; consider implementing all sampling logic in one masker"
            )
        self.maskers = maskers
        self._plan_kind = plan_kind(maskers)
        self._plans: Dict[Any, DecodePlan] = {}
        self._mask_facts = AdditiveMaskFacts()

    def _planned_capacity(self, dims) -> Optional[int]:
        """Entries per row the whole chain can add, if every masker can tell without the device."""
        total = 0
        for masker in self.maskers:
            n = masker.max_new_entries(dims)
            if n is None:
                return None
            total += n
        return total

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
        """(attention output (B, Lq, Hq, D), attention weights (B, Hq, Lq, Lk) or None)."""
        if "sparse_meta_data" not in kwargs:
            raise ValueError("sparse_meta_data must be provided in kwargs while calling custom_attention()")
        sparse_meta_data: Dict[Any, Any] = kwargs.pop("sparse_meta_data")

        if (attention_mask is not None and attention_mask.is_cuda and attention_mask.dim() == 4
                and attention_mask.shape[-1] >= keys.shape[2] and attention_mask.dtype in (torch.float32, torch.bfloat16, torch.float16)
                and self._mask_facts.all_zero(attention_mask)):
            # an additive mask of zeros (HuggingFace's eager mask of an unpadded decode step) adds nothing anywhere:
            # established once per mask tensor, i.e. once per forward pass, not per layer
            attention_mask = None

        metrics = MicroMetricLogger()
        want_density = metrics.is_metric_enabled("research_attention_density")
        want_error = metrics.is_metric_enabled("research_attention_output_error")

        if (not (want_density or want_error)  # the metrics read the finished mask: masker-by-masker path
                and not self.return_attention_weights and attention_mask is None and self._plan_kind is not None
                and not isinstance(kwargs.get("s_aux"), torch.Tensor) and queries.dim() == 4
                and not (dropout > 0.0 and module is not None and getattr(module, "training", False))):
            # decode fast path: the whole chain as one native call over cached argument blocks
            _native.require_device(queries, "queries")
            key = (queries.device, queries.dtype, tuple(queries.shape), keys.shape[1])
            plan = self._plans.get(key)
            if plan is None:
                plan = self._plans[key] = DecodePlan(self.maskers, self._plan_kind, queries, keys)
            out = plan.run(queries, keys, values, scaling, sparse_meta_data, kwargs.get("layer_idx"))
            if out is not None:
                return out, None

        mask_shape = (queries.shape[0], queries.shape[1], queries.shape[2], keys.shape[2])
        mask = Mask.create_empty_mask(mask_shape, dtype=queries.dtype, device=queries.device)
        if self.maskers:
            # size the row buffers once for the whole chain so no masker has to grow them
            dims = self.maskers[0]._extract_tensor_dimensions(keys, queries)
            planned = self._planned_capacity(dims)
            if planned is not None and planned > 0:
                rows = NativeRows(mask_shape[0] * mask_shape[1] * mask_shape[2], mask_shape[3], planned, queries.device)
                mask = _EmptyRowsMask(mask_shape, rows, queries.dtype)

        maskers = self.maskers
        if (len(maskers) >= 2 and type(maskers[0]) is SinkMasker and type(maskers[1]) is LocalMasker
                and not mask.is_full_mask()):
            # Sink directly followed by Local on a still-empty mask: one fused launch writes both ranges
            mask = fused_sink_local(maskers[0], maskers[1], keys, queries, mask)
            maskers = maskers[2:]

        # per-call scratch the maskers may share (e.g. the QK score keys of one scoring pass)
        call_scratch: Dict[str, Any] = {}
        for masker in maskers:
            mask = masker.add_mask(
                keys=keys,
                queries=queries,
                values=values,
                attention_mask=attention_mask,
                scaling=scaling,
                dropout=dropout,
                sparse_meta_data=sparse_meta_data,
                previous_mask=mask,
                _call_scratch=call_scratch,
                **kwargs,
            )

        if want_density:
            # active fraction of the (B, Hq, Lq, Lk) mask, from the per-row counts (reference :121-126)
            metrics.log("research_attention_density", mask.get_density(), metadata={"layer_idx": kwargs["layer_idx"]})

        s_aux_raw: Any = kwargs.pop("s_aux", None)
        s_aux: Optional[torch.Tensor] = s_aux_raw if isinstance(s_aux_raw, torch.Tensor) else None
        weights: Optional[torch.Tensor] = None
        # a masker of this call scored every key exactly (OracleTopK, AdaptiveSampling): the attention takes its
        # logits from those scores instead of reading K again
        kwargs["_score_keys"] = (call_scratch.get("qk_score_keys"), call_scratch.get("qk_score_resid"))
        if self.return_attention_weights:
            out, weights = get_masked_attention_output(
                module=module, queries=queries, keys=keys, values=values, attention_mask=attention_mask,
                sinks=s_aux, scaling=scaling, dropout=dropout, sparse_attention_mask=mask,
                return_attention_weights=True, **kwargs,
            )
        else:
            out = get_masked_attention_output(
                module=module, queries=queries, keys=keys, values=values, attention_mask=attention_mask,
                sinks=s_aux, scaling=scaling, dropout=dropout, sparse_attention_mask=mask,
                return_attention_weights=False, **kwargs,
            )
        if want_error:
            # relative distance to dense attention over all keys, by the same kernel in dense mode (reference :150-168)
            true_out, _ = get_true_attention_output(module, queries, keys, values, attention_mask, scaling, dropout, **kwargs)
            error = torch.norm(true_out.float() - out.float()) / torch.norm(true_out.float())
            metrics.log("research_attention_output_error", float(error.item()), metadata={"layer_idx": kwargs["layer_idx"]})
        return out, weights

    @classmethod
    def create_from_config(cls, config: SparseAttentionConfig) -> "ResearchAttention":
        if not isinstance(config, ResearchAttentionConfig):
            raise TypeError(f"Expected ResearchAttentionConfig, got {type(config)}")
        maskers = [ResearchMasker.create_masker_from_config(c) for c in config.masker_configs]
        return cls(config, maskers)


class _EmptyRowsMask(Mask):
    """An empty mask that already owns row buffers sized for the chain: it reports
    is_empty (so consumers treat it as "no masking") until a masker fills the rows."""

    def __init__(self, shape, rows: NativeRows, dtype: torch.dtype):
        super().__init__(shape=shape, dtype=dtype, device=rows.device, is_empty=True)
        self._planned_rows = rows

    def to_rows(self, extra: int = 0, weighted: Optional[bool] = None) -> NativeRows:
        rows = self._planned_rows
        rows.reserve(extra)
        if weighted:
            rows.zero_if_fresh()
            rows.make_weighted()
        return rows
