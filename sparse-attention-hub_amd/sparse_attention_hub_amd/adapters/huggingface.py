"""HuggingFace adapter: registers ResearchAttention as an attention function and drives a greedy
prefill / question / decode loop.

Reference: sparse_attention_hub/adapters/huggingface.py. What is mirrored here is the part of the
adapter that touches the attention path:
  * get_custom_attention_function (:227-275): the callable HuggingFace invokes per attention layer;
    it takes `layer_idx` from the module, requires `sparse_meta_data` among the forward kwargs and
    hands everything to `SparseAttention.custom_attention`;
  * _generate_unique_attention_name / _ensure_attention_registered / _cleanup_attention_registration
    (:277-343): registration under a fresh name in ALL_ATTENTION_FUNCTIONS, with `eager_mask` as the
    mask function of that name;
  * enable_sparse_mode (:345-385): `config._attn_implementation` switched for the duration of a block;
  * process_request / _generate_response (:106-202, :387-484): the context is prefilled with the model's
    own dense attention, then - in sparse mode - the question tokens in one pass (Lq > 1) and a greedy
    decode, one token at a time, `sparse_meta_data` carried through every forward call.
The reference's adapter also owns a model server, a tokenizer and a request type; those are outside the
attention path. This adapter takes a loaded model and token ids instead (`process_tokens`).
"""
from __future__ import annotations

import random
import string
from contextlib import contextmanager
from typing import Any, Callable, Dict, Generator, List, Optional, Sequence, Tuple

import torch

from ..sparse_attention import ResearchAttention, SparseAttention, SparseAttentionConfig


class ModelAdapterHF:
    """Wraps a HuggingFace causal LM whose attention layers go through the attention-function registry."""

    def __init__(self, model: torch.nn.Module, sparse_attention_config: Optional[SparseAttentionConfig],
                 hybrid: bool = False) -> None:
        self.model = model
        self.sparse_attention_config = sparse_attention_config
        self._sparse_attention_available: bool = sparse_attention_config is not None
        self.sparse_attention: Optional[SparseAttention] = (
            SparseAttention.create_from_config(sparse_attention_config) if sparse_attention_config is not None else None
        )
        if isinstance(self.sparse_attention, ResearchAttention):
            # HuggingFace drops the attention probabilities unless output_attentions is set
            self.sparse_attention.return_attention_weights = False
        # feed the question one token at a time (the reference does so for hybrid linear-attention models)
        self.hybrid = hybrid
        self._registered_attention_name: Optional[str] = None
        self._custom_attention_fn: Optional[Callable] = None

    def __del__(self) -> None:
        try:
            self._cleanup_attention_registration()
        except Exception:
            pass

    # ------------------------------------------------------------------ the attention callable
    def get_custom_attention_function(self, sparse_attention: SparseAttention) -> Callable:
        def custom_attention_callable(module: torch.nn.Module, queries: torch.Tensor, keys: torch.Tensor,
                                      values: torch.Tensor, attention_mask: Optional[torch.Tensor],
                                      scaling: float = 1.0, dropout: float = 0.0,
                                      **kwargs: Dict[str, Any]) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
            if hasattr(module, "layer_idx"):
                layer_idx = getattr(module, "layer_idx", None)
                if layer_idx is not None:
                    kwargs["layer_idx"] = layer_idx
            if "sparse_meta_data" in kwargs:
                sparse_meta_data: Dict[Any, Any] = kwargs.pop("sparse_meta_data")
            else:
                raise ValueError("sparse_meta_data must be provided while calling model.forward()")
            return sparse_attention.custom_attention(
                module=module, queries=queries, keys=keys, values=values, attention_mask=attention_mask,
                scaling=scaling, dropout=dropout, sparse_meta_data=sparse_meta_data, **kwargs,
            )

        return custom_attention_callable

    # ------------------------------------------------------------------ registration
    @staticmethod
    def _registries():
        from transformers.masking_utils import ALL_MASK_ATTENTION_FUNCTIONS
        from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

        return ALL_ATTENTION_FUNCTIONS, ALL_MASK_ATTENTION_FUNCTIONS

    def _generate_unique_attention_name(self) -> str:
        attn, mask = self._registries()
        existing: List[str] = list(attn.valid_keys()) + list(mask.valid_keys())
        while True:
            suffix = "".join(random.choices(string.ascii_lowercase + string.digits, k=8))
            name = f"sparse_attention_{suffix}"
            if name not in existing:
                return name

    def _ensure_attention_registered(self) -> str:
        if self._registered_attention_name is None:
            if not self._sparse_attention_available or self.sparse_attention is None:
                raise RuntimeError("Cannot register attention function: sparse attention is not available")
            self._custom_attention_fn = self.get_custom_attention_function(self.sparse_attention)
            self._registered_attention_name = self._generate_unique_attention_name()
            from transformers.masking_utils import eager_mask

            attn, mask = self._registries()
            attn.register(self._registered_attention_name, self._custom_attention_fn)
            if isinstance(self.sparse_attention, ResearchAttention):
                mask.register(self._registered_attention_name, eager_mask)
            else:
                raise NotImplementedError("Sparse attention is not supported for this model yet")
        return self._registered_attention_name

    def _cleanup_attention_registration(self) -> None:
        name = self._registered_attention_name
        if name is not None:
            attn, mask = self._registries()
            for registry in (attn, mask):
                if name in registry.valid_keys():
                    registry._global_mapping.pop(name, None)
        self._registered_attention_name = None
        self._custom_attention_fn = None

    @contextmanager
    def enable_sparse_mode(self) -> Generator[None, None, None]:
        if not self._sparse_attention_available:
            raise RuntimeError("Cannot enable sparse mode: sparse attention is not available")
        original: Dict[str, str] = {}
        for name, module in self.model.named_modules():
            if hasattr(module, "config") and hasattr(module.config, "_attn_implementation"):
                original[name] = module.config._attn_implementation
        custom_name = self._ensure_attention_registered()
        try:
            for name, module in self.model.named_modules():
                if hasattr(module, "config") and hasattr(module.config, "_attn_implementation"):
                    module.config._attn_implementation = custom_name
            yield
        finally:
            for name, module in self.model.named_modules():
                if name in original:
                    module.config._attn_implementation = original[name]

    # ------------------------------------------------------------------ generation
    def _generate_tokens(self, question_tokens: torch.Tensor, context_outputs: Any, sparse_meta_data: Dict[str, Any],
                         max_new_tokens: int, stop_token_ids: Sequence[int] = ()) -> torch.Tensor:
        """Greedy continuation after the context prefill — the token-id form of _generate_response."""
        past = context_outputs.past_key_values
        last = None

        def forward(ids: torch.Tensor, **extra: Any):
            kwargs: Dict[str, Any] = {"input_ids": ids, "past_key_values": past, "use_cache": True}
            kwargs.update(extra)
            if self._sparse_attention_available:
                kwargs["sparse_meta_data"] = sparse_meta_data
            with torch.no_grad():
                return self.model(**kwargs)

        if self.hybrid:
            for idx in range(question_tokens.shape[1]):
                last = forward(question_tokens[:, idx: idx + 1], logits_to_keep=1)
                past = last.past_key_values
        else:
            last = forward(question_tokens)
            past = last.past_key_values
        if last is None:
            raise ValueError("Question tokens are empty; cannot generate response")
        generated = [last.logits[0, -1].argmax()]
        for _ in range(max_new_tokens - 1):
            out = forward(generated[-1].unsqueeze(0).unsqueeze(0))
            past = out.past_key_values
            new_id = out.logits[0, -1].argmax()
            generated.append(new_id)
            if stop_token_ids and int(new_id.item()) in stop_token_ids:
                break
        return torch.stack(generated)

    def process_tokens(self, context_tokens: torch.Tensor, questions: Sequence[torch.Tensor], max_new_tokens: int,
                       stop_token_ids: Sequence[int] = ()) -> List[torch.Tensor]:
        """The token-id form of process_request: the context is prefilled once per question with the model's own
        attention, each question is answered independently (fresh sparse_meta_data, fresh KV cache)."""
        self.model.eval()
        answers: List[torch.Tensor] = []
        with torch.no_grad():
            for question_tokens in questions:
                sparse_meta_data: Dict[str, Any] = {}
                if self._sparse_attention_available:
                    context_outputs = self.model(context_tokens, past_key_values=None, use_cache=True,
                                                 sparse_meta_data=sparse_meta_data)
                    with self.enable_sparse_mode():
                        answers.append(self._generate_tokens(question_tokens, context_outputs, sparse_meta_data,
                                                             max_new_tokens, stop_token_ids))
                else:
                    context_outputs = self.model(context_tokens, past_key_values=None, use_cache=True)
                    answers.append(self._generate_tokens(question_tokens, context_outputs, sparse_meta_data,
                                                         max_new_tokens, stop_token_ids))
        return answers
