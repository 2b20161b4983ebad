"""HashAttention weight containers.

File layout of the reference (sparse_attention/utils/hashattention_utils.py:155-180):
a pickle of Dict[layer_idx] -> {"query_matrix", "query_bias", "key_matrix",
"key_bias"} -> List[Tensor], matrices (H, d_in, d_out) and biases (H, d_out), one
list entry per MLP layer.
"""
from __future__ import annotations

import collections
import io
import pickle
from typing import Dict, List

import torch

HatWeights = Dict[int, Dict[str, List[torch.Tensor]]]


def _storage_from_bytes(data: bytes):
    """What `torch.storage._load_from_bytes` does for a pickled tensor's storage, but through the loader that
    executes nothing from the bytes."""
    return torch.load(io.BytesIO(data), weights_only=True)


class _HatUnpickler(pickle.Unpickler):
    """Unpickler that resolves only what a dict of lists of CPU tensors needs. A tensor pickles as
    `torch._utils._rebuild_tensor_v2(storage, ...)` with the storage as `torch.storage._load_from_bytes(bytes)`
    (replaced here by the safe loader above) and its (empty) hooks as an OrderedDict; `nn.Parameter`s add
    `_rebuild_parameter`. Every other global a file asks for is refused, so loading runs no code from the file."""

    _ALLOWED = {
        ("torch._utils", "_rebuild_tensor_v2"): lambda: torch._utils._rebuild_tensor_v2,
        ("torch._utils", "_rebuild_parameter"): lambda: torch._utils._rebuild_parameter,
        ("torch.storage", "_load_from_bytes"): lambda: _storage_from_bytes,
        ("collections", "OrderedDict"): lambda: collections.OrderedDict,
    }

    def find_class(self, module: str, name: str):
        try:
            return self._ALLOWED[(module, name)]()
        except KeyError:
            raise pickle.UnpicklingError(
                f"HAT weight file refers to {module}.{name}; only plain containers of tensors are accepted") from None


def load_hat_weights(hat_weights_path: str, device: str = "cpu") -> HatWeights:
    """Load a HAT weight pickle written by this package or by the reference tools
    (reference: hashattention_utils.py:155-180). The file is read with an allow-list unpickler: anything but
    dicts, lists, numbers, strings and tensors raises `pickle.UnpicklingError`."""
    with open(hat_weights_path, "rb") as f:
        hat_weights = _HatUnpickler(f).load()
    if not isinstance(hat_weights, dict):
        raise ValueError(f"{hat_weights_path}: expected Dict[layer] -> Dict[name] -> List[Tensor], got {type(hat_weights).__name__}")
    for layer_idx, layer_weights in hat_weights.items():
        if not isinstance(layer_weights, dict):
            raise ValueError(f"{hat_weights_path}: layer {layer_idx!r} is not a dict")
        for name, tensors in layer_weights.items():
            if not all(isinstance(t, torch.Tensor) for t in tensors):
                raise ValueError(f"{hat_weights_path}: layer {layer_idx!r} entry {name!r} holds non-tensors")
            hat_weights[layer_idx][name] = [t.detach().to(device) for t in tensors]
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


def convert_usa_weights_to_hash_attention(usa_checkpoint, num_layers: int = 32, num_heads: int = 32,
                                          num_mlp_layers: int = 3, device: str = "cpu") -> HatWeights:
    """USA-module weights -> the HashAttention layout (reference: hashattention_utils.py:9-116).

    `usa_checkpoint` is a state dict or the path of one (read with torch.load(..., weights_only=True), which
    executes nothing from the file). Its entries are the per-head torch.nn.Sequential MLPs of the USA module,
    `{layer}.learning_to_hash_transformation_{q|k}.{head}.{2 i}.{weight|bias}` for MLP layer i (the odd indices are
    the activations). nn.Linear stores (out, in): matrices are transposed to (in, out) and stacked over the heads;
    a missing bias becomes zeros. Layers or heads absent from the checkpoint are skipped, like in the reference."""
    if isinstance(usa_checkpoint, (str, bytes)) or hasattr(usa_checkpoint, "__fspath__"):
        state = torch.load(usa_checkpoint, map_location=device, weights_only=True)
    else:
        state = usa_checkpoint
    hat_weights: HatWeights = {}
    for layer_idx in range(num_layers):
        layer: Dict[str, List[torch.Tensor]] = {"query_matrix": [], "query_bias": [], "key_matrix": [], "key_bias": []}
        for i in range(num_mlp_layers):
            per_kind = {}
            for kind, tag in (("query", "q"), ("key", "k")):
                mats, biases = [], []
                for head in range(num_heads):
                    prefix = f"{layer_idx}.learning_to_hash_transformation_{tag}.{head}.{2 * i}"
                    weight = state.get(f"{prefix}.weight")
                    if weight is None:
                        continue
                    mats.append(weight.t().to(device))
                    bias = state.get(f"{prefix}.bias")
                    biases.append(torch.zeros(weight.shape[0], device=device) if bias is None else bias.to(device))
                per_kind[kind] = (mats, biases)
            if per_kind["query"][0]:
                layer["query_matrix"].append(torch.stack(per_kind["query"][0]))
                layer["query_bias"].append(torch.stack(per_kind["query"][1]))
                layer["key_matrix"].append(torch.stack(per_kind["key"][0]))
                layer["key_bias"].append(torch.stack(per_kind["key"][1]))
        hat_weights[layer_idx] = layer
    return hat_weights


def create_hat_weights_file_from_usa(usa_checkpoint, target_hat_path: str, num_layers: int = 32, num_heads: int = 32,
                                     num_mlp_layers: int = 3, device: str = "cpu") -> None:
    """Convert and save in the reference's HAT file format (hashattention_utils.py:119-152)."""
    save_hat_weights(convert_usa_weights_to_hash_attention(usa_checkpoint, num_layers, num_heads, num_mlp_layers, device),
                     target_hat_path)
