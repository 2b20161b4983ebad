"""HashAttention top-k masker on packed bit signatures.

Reference (maskers/fixed/implementations/hashattention_top_k.py): keys (after
repeat_kv, so per *query* head) and queries go through a per-head MLP, `sign`
gives +-1 float signatures (:203-238) that are cached per layer in
sparse_meta_data["key"] (:255-341); scores = q_sig @ k_sig^T (:365-367), active
columns are pushed to the bottom and torch.topk picks heavy_size columns
(fixed/base.py:74-85), merged into the previous mask.

Here a signature is two uint32 planes (bit e of plane 0 = output e > 0, of plane 1
= output e != 0; exact zeros do occur in bf16 and the reference scores them as
0), the cache is a packed [B, Hq, capacity, 2] buffer that grows in place, the
score is popcount(nz) - 2 * popcount((q ^ k) & nz), and `sah_hamming_topk` fuses
scoring, selection with the lowest-column tie rule and the merge into the row
lists.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from .....utils.hashattention_utils import load_hat_weights
from .....utils.kv_utils import _get_num_key_value_groups
from .....utils.mask import Mask
from .....utils.mask_attention_utils import _inner_contiguous, additive_mask_args
from ...... import _native as N
from ...base import AttentionTensorDimensions, MaskerConfig, MaskerRegistry
from ..base import TopKMasker, TopKMaskerConfig, sortable_key_of
from .oracle_top_k import _default_search_space, score_key_buffer


@dataclass
class HashAttentionTopKMaskerConfig(TopKMaskerConfig):
    hat_bits: int
    hat_mlp_layers: int
    hat_mlp_hidden_size: int
    hat_mlp_activation: str
    hat_weights: Optional[Dict[int, Dict[str, List[torch.Tensor]]]] = None
    hat_weight_file: Optional[str] = None
    search_space: Dict[str, Any] = field(default_factory=_default_search_space)


class PackedSignatureCache:
    """Key signatures of one layer: int32 codes [B, Hq, capacity, 2] (positive plane,
    non-zero plane), `n` of them valid.

    Stands where the reference keeps a float tensor (B, Hq, n, bits) in
    sparse_meta_data["key"][layer]; `.shape` reports that logical shape and
    `unpack()` rebuilds the +-1 float tensor for callers that want it.
    """

    def __init__(self, batch: int, heads: int, bits: int, capacity: int, device: torch.device):
        self.bits = bits
        self.n = 0
        capacity = (capacity + 63) // 64 * 64  # rows of codes stay 16-byte aligned for the vector loads
        self.codes = torch.empty((batch, heads, capacity, 2), dtype=torch.int32, device=device)
        # compact form for the decode kernel (built on demand by `compact_upto`): sign planes [B, Hq, pos_pitch],
        # columns with a zero component [B, Hq, exc_cap, 4] and their number [B, Hq]; valid for `n_compact` keys
        self.pos = self.exc = self.exc_cnt = None
        self.n_compact = 0

    @property
    def capacity(self) -> int:
        return self.codes.shape[2]

    @property
    def shape(self) -> Tuple[int, int, int, int]:
        return (self.codes.shape[0], self.codes.shape[1], self.n, self.bits)

    def reserve(self, n_total: int) -> None:
        if n_total <= self.capacity:
            return
        new_cap = (max(n_total + 4096, 2 * self.capacity) + 63) // 64 * 64
        grown = torch.empty((self.codes.shape[0], self.codes.shape[1], new_cap, 2), dtype=torch.int32, device=self.codes.device)
        if self.n:
            grown[:, :, : self.n] = self.codes[:, :, : self.n]
        self.codes = grown
        self.pos = self.exc = self.exc_cnt = None  # rebuilt from the codes at the next decode step
        self.n_compact = 0

    @property
    def full_plane(self) -> int:
        return (1 << self.bits) - 1

    def ensure_compact_buffers(self) -> None:
        """Buffers of the compact form, sized for the current capacity (8192 columns of slack for the
        kernel's whole-chunk reads)."""
        if self.pos is not None:
            return
        B, H = self.codes.shape[0], self.codes.shape[1]
        dev = self.codes.device
        pitch = self.capacity + 8192
        self.pos = torch.zeros((B, H, pitch), dtype=torch.int32, device=dev)
        self.exc = torch.empty((B, H, max(1024, self.capacity // 16), 4), dtype=torch.int32, device=dev)
        self.exc_cnt = torch.zeros((B, H), dtype=torch.int32, device=dev)
        self.n_compact = 0

    def unpack(self, dtype: torch.dtype = torch.float32) -> torch.Tensor:
        codes = self.codes[:, :, : self.n].to(torch.int64) & 0xFFFFFFFF
        shifts = torch.arange(self.bits, device=codes.device, dtype=torch.int64)
        pos = (codes[..., 0].unsqueeze(-1) >> shifts) & 1
        nonzero = (codes[..., 1].unsqueeze(-1) >> shifts) & 1
        return ((pos * 2 - 1) * nonzero).to(dtype)


@MaskerRegistry.register(HashAttentionTopKMaskerConfig)
class HashAttentionTopKMasker(TopKMasker):
    heavy_size: Union[float, int]
    hat_bits: int
    hat_mlp_layers: int
    hat_mlp_hidden_size: int
    hat_mlp_activation: str
    hat_weights: Dict[int, Dict[str, List[torch.Tensor]]]

    def __init__(self, config: HashAttentionTopKMaskerConfig) -> None:
        super().__init__(config)
        self.heavy_size = config.heavy_size
        self.hat_bits = config.hat_bits
        self.hat_mlp_layers = config.hat_mlp_layers
        self.hat_mlp_hidden_size = config.hat_mlp_hidden_size
        self.hat_mlp_activation = config.hat_mlp_activation
        if config.hat_weights is not None and config.hat_weight_file is not None:
            raise ValueError("Only one of hat_weights or hat_weight_file should be provided")
        if config.hat_weights is None and config.hat_weight_file is None:
            raise ValueError("Either hat_weights or hat_weight_file must be provided")
        if config.hat_weight_file is not None:
            self.hat_weights = load_hat_weights(config.hat_weight_file)
        else:
            self.hat_weights = config.hat_weights
        # (layer, kind, device, dtype) -> (matrices, biases) laid out for the kernel, built once
        self._prepared: Dict[Tuple[int, str, str, torch.dtype], Tuple[List[torch.Tensor], List[torch.Tensor]]] = {}

    # ---------------------------------------------------------------- helpers
    def _validate_inputs(self, sparse_meta_data, kwargs: Dict[str, Any]) -> int:
        if sparse_meta_data is None:
            raise ValueError("sparse_meta_data cannot be None")
        layer_idx = kwargs.get("layer_idx")
        if layer_idx is None:
            raise ValueError("layer_idx must be provided in kwargs")
        return layer_idx

    def _calculate_effective_heavy_size(self, seq_len_keys: int) -> int:
        return self._calculate_effective_size(self.heavy_size, seq_len_keys)

    def _should_use_full_attention(self, dims: AttentionTensorDimensions, heavy_size: int) -> bool:
        return dims.seq_len_keys <= heavy_size

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        return self._calculate_effective_heavy_size(dims.seq_len_keys)

    def _weights_for(self, layer_idx: int, kind: str, device: torch.device, dtype: torch.dtype):
        key = (layer_idx, kind, str(device), dtype)
        hit = self._prepared.get(key)
        if hit is not None:
            return hit
        layer = self.hat_weights[layer_idx]
        mats = [m.to(device=device, dtype=dtype).contiguous() for m in layer[f"{kind}_matrix"]]
        biases = [b.to(device=device, dtype=dtype).contiguous() for b in layer[f"{kind}_bias"]]
        if not mats:
            raise ValueError("hat_weights hold no MLP layers")
        if len(mats) > N.SAH_MAX_MLP_LAYERS:
            raise ValueError(f"at most {N.SAH_MAX_MLP_LAYERS} signature MLP layers are supported, got {len(mats)}")
        if self.hat_mlp_activation not in N.SAH_ACT:
            raise ValueError(f"Unsupported activation function: {self.hat_mlp_activation}")
        # the same matrices transposed to [heads, d_out, d_in]: the matrix-core path of the bulk kernel reads them
        mats_t = [m.transpose(1, 2).contiguous() for m in mats]
        self._prepared[key] = (mats, biases, mats_t)
        return mats, biases, mats_t

    def _hash_args(self, x: torch.Tensor, x_heads: int, n_heads: int, first: int, count: int, layer_idx: int,
                   kind: str, codes: torch.Tensor, code_pitch: int, code_offset: int) -> "N.HashSigArgs":
        """Argument block for the signatures of x[:, :, first:first+count, :] into codes[..., code_offset:]."""
        mats, biases, mats_t = self._weights_for(layer_idx, kind, x.device, x.dtype)
        if mats[0].shape[0] != n_heads or mats[0].shape[1] != x.shape[-1]:
            raise ValueError(
                f"{kind}_matrix[0] has shape {tuple(mats[0].shape)}, expected ({n_heads}, {x.shape[-1]}, *)"
            )
        W = (N.C.c_void_p * N.SAH_MAX_MLP_LAYERS)()
        Bv = (N.C.c_void_p * N.SAH_MAX_MLP_LAYERS)()
        Wt = (N.C.c_void_p * N.SAH_MAX_MLP_LAYERS)()
        dout = (N.C.c_int32 * N.SAH_MAX_MLP_LAYERS)()
        for i, (m, b, mt) in enumerate(zip(mats, biases, mats_t)):
            W[i], Bv[i], Wt[i], dout[i] = m.data_ptr(), b.data_ptr(), mt.data_ptr(), m.shape[2]
        args = N.HashSigArgs(
            x.data_ptr() + first * x.stride(2) * x.element_size(),
            x.stride(0), x.stride(1), x.stride(2),
            N.dtype_code(x.dtype),
            x.shape[0], n_heads, n_heads // x_heads, count, x.shape[-1],
            len(mats), W, Bv, Wt, dout, N.SAH_ACT[self.hat_mlp_activation],
            codes.data_ptr(), code_pitch, code_offset, N.stream_ptr(x.device),
        )
        args._keepalive = (W, Bv, Wt, dout)
        return args

    def _hash(self, x: torch.Tensor, x_heads: int, n_heads: int, first: int, count: int, layer_idx: int,
              kind: str, codes: torch.Tensor, code_pitch: int, code_offset: int) -> None:
        """Signatures of x[:, :, first:first+count, :] into codes[..., code_offset:]."""
        if count <= 0:
            return
        N.call("sah_hash_signatures",
               self._hash_args(x, x_heads, n_heads, first, count, layer_idx, kind, codes, code_pitch, code_offset))

    def _update_key_signatures(self, keys: torch.Tensor, n_heads: int, sparse_meta_data, layer_idx: int,
                               pair_with=None) -> PackedSignatureCache:
        """Hash only the keys beyond the cached count and append them (reference :255-341).
        pair_with=(queries, qcodes): also hash the queries, in the same launch when both jobs are small."""
        cache_map = sparse_meta_data.setdefault("key", {})
        cache = cache_map.get(layer_idx)
        B, Hkv, Lk = keys.shape[0], keys.shape[1], keys.shape[2]
        if cache is None:
            cache = PackedSignatureCache(B, n_heads, self.hat_bits, Lk + 4096, keys.device)
            cache_map[layer_idx] = cache
        if Lk < cache.n:
            raise ValueError(f"Current number of keys ({Lk}) is less than cached number of keys ({cache.n})")
        qargs = None
        if pair_with is not None:
            q, qcodes = pair_with
            qargs = self._hash_args(q, n_heads, n_heads, 0, q.shape[2], layer_idx, "query", qcodes, q.shape[2], 0)
        if Lk > cache.n:
            cache.reserve(Lk)
            kargs = self._hash_args(keys, Hkv, n_heads, cache.n, Lk - cache.n, layer_idx, "key", cache.codes,
                                    cache.capacity, cache.n)
            if qargs is not None:
                N.call2("sah_hash_signatures_pair", kargs, qargs)
                qargs = None
            else:
                N.call("sah_hash_signatures", kargs)
            cache.n = Lk
        if qargs is not None:
            N.call("sah_hash_signatures", qargs)
        return cache

    # ------------------------------------------------------------------- main
    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        layer_idx = self._validate_inputs(sparse_meta_data, kwargs)
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
        Lk = keys.shape[2]
        q = _inner_contiguous(queries)
        k = _inner_contiguous(keys)

        qcodes = torch.empty((B * Hq * Lq, 2), dtype=torch.int32, device=q.device)
        cache = self._update_key_signatures(k, Hq, sparse_meta_data, layer_idx, pair_with=(q, qcodes))

        rows = previous_mask.to_rows(extra=k_eff)
        rows.zero_if_fresh()
        if attention_mask is None:
            args = N.HammingTopkArgs(rows.as_struct(), cache.codes.data_ptr(), cache.capacity, qcodes.data_ptr(),
                                     Lq, k_eff, N.stream_ptr(q.device))
            N.call("sah_hamming_topk", args)
            rows.note_added(k_eff, exact=(Lk - rows.max_cnt >= k_eff))
        else:
            keybuf = score_key_buffer(rows.n_rows, Lk, q.dtype, q.device)
            am_keep, am_ptr, ms_b, ms_h, ms_l = additive_mask_args(attention_mask, q, Lk)
            sargs = N.HammingScoresArgs(
                cache.codes.data_ptr(), cache.capacity, qcodes.data_ptr(), B, Hq, Lq, Lk,
                am_ptr, ms_b, ms_h, ms_l, N.dtype_code(q.dtype), keybuf.data_ptr(), keybuf.stride(0),
                N.stream_ptr(q.device),
            )
            N.call("sah_hamming_scores", sargs)
            excluded = sortable_key_of(float("-inf"), q.dtype)
            self._select_into_rows(rows, keybuf, 32 if q.dtype == torch.float32 else 16, Lk, 0, k_eff, excluded)
        return Mask.create_mask_from_rows(self._mask_shape(dims), rows, previous_mask.dtype)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "HashAttentionTopKMasker":
        if not isinstance(config, HashAttentionTopKMaskerConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)
