"""HashAttention weight containers.

File layout of the reference (sparse_attention/utils/hashattention_utils.py:155-180):
a pickle of Dict[layer_idx] -> {"query_matrix", "query_bias", "key_matrix",
"key_bias"} -> List[Tensor], matrices (H, d_in, d_out) and biases (H, d_out), one
list entry per MLP layer.
"""
from __future__ import annotations

import pickle
from typing import Dict, List

import torch

HatWeights = Dict[int, Dict[str, List[torch.Tensor]]]


def load_hat_weights(hat_weights_path: str, device: str = "cpu") -> HatWeights:
    """Load a HAT weight pickle written by this package or by the reference tools.

    Pickles execute code on load: only open files you wrote or trust."""
    with open(hat_weights_path, "rb") as f:
        hat_weights: HatWeights = pickle.load(f)
    for layer_idx, layer_weights in hat_weights.items():
        for name, tensors in layer_weights.items():
            hat_weights[layer_idx][name] = [t.to(device) for t in tensors]
    return hat_weights


def save_hat_weights(hat_weights: HatWeights, path: str) -> None:
    cpu = {
        layer: {name: [t.detach().cpu() for t in tensors] for name, tensors in weights.items()}
        for layer, weights in hat_weights.items()
    }
    with open(path, "wb") as f:
        pickle.dump(cpu, f)


def random_hat_weights(
    num_layers: int,
    num_heads: int,
    head_dim: int,
    hat_bits: int,
    hat_mlp_layers: int,
    hat_mlp_hidden_size: int,
    dtype: torch.dtype = torch.float32,
    seed: int = 0,
    device: str = "cpu",
) -> HatWeights:
    """Random-init signature MLPs: W ~ N(0, 1/fan_in), b ~ N(0, 1/fan_in)."""
    gen = torch.Generator().manual_seed(seed)
    dims = [head_dim] + [hat_mlp_hidden_size] * (hat_mlp_layers - 1) + [hat_bits]
    out: HatWeights = {}
    for layer in range(num_layers):
        entry: Dict[str, List[torch.Tensor]] = {"query_matrix": [], "query_bias": [], "key_matrix": [], "key_bias": []}
        for kind in ("query", "key"):
            for i in range(hat_mlp_layers):
                std = dims[i] ** -0.5
                w = torch.randn(num_heads, dims[i], dims[i + 1], generator=gen) * std
                b = torch.randn(num_heads, dims[i + 1], generator=gen) * std
                entry[f"{kind}_matrix"].append(w.to(dtype).to(device))
                entry[f"{kind}_bias"].append(b.to(dtype).to(device))
        out[layer] = entry
    return out
