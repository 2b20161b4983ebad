"""GQA helpers (reference: sparse_attention/utils/kv_utils.py:5-45).

The kernels map query head h to KV head h // groups by index arithmetic and never
materialise the repeated tensor; `repeat_kv` is kept for callers that want the
expanded view.
"""
import torch


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(B, Hkv, L, D) -> (B, Hkv * n_rep, L, D); each KV head repeated n_rep times in a row."""
    if n_rep == 1:
        return hidden_states
    return torch.repeat_interleave(hidden_states, repeats=n_rep, dim=1)


def _get_num_key_value_groups(queries: torch.Tensor, kv_tensor: torch.Tensor) -> int:
    """Hq // Hkv; ValueError when Hq is not a multiple of Hkv."""
    num_attention_heads: int = queries.shape[1]
    num_key_value_heads: int = kv_tensor.shape[1]
    if num_attention_heads % num_key_value_heads != 0:
        raise ValueError(
            f"num_attention_heads ({num_attention_heads}) must be divisible by num_key_value_heads ({num_key_value_heads})"
        )
    return num_attention_heads // num_key_value_heads
