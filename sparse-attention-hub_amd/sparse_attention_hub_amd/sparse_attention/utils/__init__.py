"""Mask type, masked-softmax attention and GQA helpers of the ResearchAttention path."""
from .kv_utils import _get_num_key_value_groups, repeat_kv
from .mask import Mask
from .mask_attention_utils import (
    apply_inv_mask_sum,
    get_masked_attention_output,
    get_true_attention_output,
)

__all__ = [
    "Mask",
    "repeat_kv",
    "_get_num_key_value_groups",
    "apply_inv_mask_sum",
    "get_masked_attention_output",
    "get_true_attention_output",
]
