"""PQCache masker: product-quantised keys, ADC scoring, top-k.

Reference (maskers/fixed/implementations/pq_top_k.py): on the first call per layer
the keys beyond `init_offset` are split into `pq_group_factor` sub-vectors and
clustered per (batch, kv head, sub-space) with batched k-means (:194-262); later
calls quantise only the new keys against the frozen centroids (:264-404); every
call scores all quantised keys through a query x centroid table and the codes
(:406-490), masks out active columns and takes the top-k (:492-537).

Here the codes are uint8 [B, Hkv, capacity, n_sub] (16 bytes per key at
n_sub=16 instead of the reference's int64 indices repeated per query head), the
lookup table lives in LDS, and selection appends to the row lists directly.
State is kept in `sparse_meta_data` under the reference's keys: "pq_centroids"
(B, Hkv, n_sub, 2^bits, d_sub) in the key dtype, "pq_codebook" (a PQCodebook),
"pq_ip2l2_phi"; plus "pq_centroids_f32", the fp32 widening the kernels read.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

import torch

from .....utils.kv_utils import _get_num_key_value_groups
from .....utils.mask import Mask
from .....utils.mask_attention_utils import _inner_contiguous
from ...... import _native as N
from ...base import AttentionTensorDimensions, MaskerConfig, MaskerRegistry
from ..base import TopKMasker, TopKMaskerConfig, sortable_key_of
from .oracle_top_k import score_key_buffer
from .utils.pq_utils import kmeans_keys_batched


@dataclass
class PQCacheConfig(TopKMaskerConfig):
    """heavy_size keys picked by PQ scores; head_dim is split into pq_group_factor sub-spaces of
    2**pq_bits centroids each; keys before init_offset are never quantised."""

    pq_group_factor: int
    pq_bits: int
    kmeans_iter: int
    init_offset: int
    metric: str

    def __post_init__(self) -> None:
        super().__post_init__()
        if self.pq_group_factor <= 0:
            raise ValueError(f"pq_group_factor must be > 0, got {self.pq_group_factor}")
        if self.pq_bits <= 0:
            raise ValueError(f"pq_bits must be > 0, got {self.pq_bits}")
        if self.kmeans_iter <= 0:
            raise ValueError(f"kmeans_iter must be > 0, got {self.kmeans_iter}")
        if self.init_offset < 0:
            raise ValueError(f"init_offset must be >= 0, got {self.init_offset}")
        if self.metric not in ["euclidean", "ip"]:
            raise ValueError(f"metric must be 'euclidean' or 'ip', got '{self.metric}'")


class PQCodebook:
    """uint8 codes [B, Hkv, capacity, n_sub], `n` keys valid; logical shape (B, n, Hkv, n_sub)
    as the reference's int64 codebook."""

    def __init__(self, batch: int, kv_heads: int, n_sub: int, capacity: int, device: torch.device):
        self.n = 0
        self.codes = torch.empty((batch, kv_heads, capacity, n_sub), dtype=torch.uint8, device=device)

    @property
    def capacity(self) -> int:
        return self.codes.shape[2]

    @property
    def shape(self) -> Tuple[int, int, int, int]:
        return (self.codes.shape[0], self.n, self.codes.shape[1], self.codes.shape[3])

    def reserve(self, n_total: int) -> None:
        if n_total <= self.capacity:
            return
        b, h, cap, s = self.codes.shape
        grown = torch.empty((b, h, max(n_total + 4096, 2 * cap), s), dtype=torch.uint8, device=self.codes.device)
        if self.n:
            grown[:, :, : self.n] = self.codes[:, :, : self.n]
        self.codes = grown

    def to_reference(self) -> torch.Tensor:
        """int64 (B, n, Hkv, n_sub), the reference's layout."""
        return self.codes[:, :, : self.n].permute(0, 2, 1, 3).to(torch.int64)


def adc_lut_buffer(B: int, Hq: int, Hkv: int, Lq: int, n_sub: int, n_cent: int, dtype: torch.dtype,
                   device: torch.device) -> torch.Tensor:
    """Scratch for the per-step lookup table of the ADC scoring (bytes)."""
    n = int(N.lib().sah_pq_adc_lut_bytes(B, Hq, Hkv, Lq, n_sub, n_cent, N.dtype_code(dtype)))
    return torch.empty((max(n, 8),), dtype=torch.uint8, device=device)


@MaskerRegistry.register(PQCacheConfig)
class PQCache(TopKMasker):
    def __init__(self, config: PQCacheConfig) -> None:
        super().__init__(config)
        self.heavy_size = config.heavy_size
        self.pq_group_factor = config.pq_group_factor
        self.pq_bits = config.pq_bits
        self.kmeans_iter = config.kmeans_iter
        self.init_offset = config.init_offset
        self.metric = config.metric
        self.kmeans_seed = 0

    def _validate_inputs(self, sparse_meta_data, kwargs: Dict[str, Any]) -> int:
        if sparse_meta_data is None:
            raise ValueError("sparse_meta_data cannot be None")
        layer_idx = kwargs.get("layer_idx")
        if layer_idx is None:
            raise ValueError("layer_idx must be provided in kwargs")
        return layer_idx

    def _should_use_full_attention(self, dims: AttentionTensorDimensions, heavy_size: int) -> bool:
        total_needed = heavy_size + self.init_offset + dims.seq_len_queries + 2 ** self.pq_bits
        return dims.seq_len_keys <= total_needed

    def max_new_entries(self, dims: AttentionTensorDimensions) -> Optional[int]:
        return self._calculate_effective_size(self.heavy_size, dims.seq_len_keys)

    def _initialize_pq_cache(self, sparse_meta_data: Dict[str, Any], layer_idx: int) -> None:
        for name in ("pq_centroids", "pq_codebook", "pq_ip2l2_phi", "pq_centroids_f32"):
            sparse_meta_data.setdefault(name, {}).setdefault(layer_idx, None)

    def _geometry(self, keys: torch.Tensor) -> Tuple[int, int, int]:
        head_dim = keys.shape[-1]
        n_sub = self.pq_group_factor
        if head_dim % n_sub:
            raise ValueError(f"head_dim {head_dim} is not divisible by pq_group_factor {n_sub}")
        if self.pq_bits > 8:
            raise ValueError(f"pq_bits {self.pq_bits} > 8: codes are stored as uint8")
        return n_sub, head_dim // n_sub, 2 ** self.pq_bits

    def _augmented(self, keys: torch.Tensor, first: int, n_sub: int, d_sub: int, phi: Optional[torch.Tensor]):
        """metric="ip": keys[:, :, first:] as (B, Hkv, n, n_sub * (d_sub + 1)) in the key dtype, every sub-vector
        followed by its extra coordinate - sqrt(phi - ||x||^2) with phi the largest squared norm of the
        (b, kv head, sub-space) group when the keys are clustered (phi=None; pq_utils.py:585-612), 0 for keys
        quantised later (pq_utils.py:615-640). Returns (augmented keys, phi [n_groups, 1, 1])."""
        B, Hkv, Lk, _ = keys.shape
        n = Lk - first
        sub = keys[:, :, first:, :].reshape(B, Hkv, n, n_sub, d_sub)
        if phi is None:
            norms_sq = (sub ** 2).sum(dim=-1, keepdim=True)
            phi5 = norms_sq.max(dim=2, keepdim=True)[0]
            extra = torch.sqrt(phi5 - norms_sq)
            phi = phi5.permute(0, 1, 3, 2, 4).reshape(-1, 1, 1)
        else:
            extra = torch.zeros((B, Hkv, n, n_sub, 1), dtype=keys.dtype, device=keys.device)
        return torch.cat([sub, extra], dim=-1).reshape(B, Hkv, n, n_sub * (d_sub + 1)).contiguous(), phi

    def _perform_kmeans_clustering(self, keys: torch.Tensor, layer_idx: int, sparse_meta_data: Dict[str, Any]):
        """First call of a layer: cluster keys[:, :, init_offset:] and store centroids + codes."""
        B, Hkv, Lk, _ = keys.shape
        n_sub, d_sub, n_cent = self._geometry(keys)
        n_keys = Lk - self.init_offset
        book = PQCodebook(B, Hkv, n_sub, n_keys + 4096, keys.device)
        source, first, d_fit = keys, self.init_offset, d_sub
        if self.metric == "ip":
            # inner-product search as L2 search: cluster the augmented sub-vectors (one more dimension)
            source, phi = self._augmented(keys, self.init_offset, n_sub, d_sub, None)
            first, d_fit = 0, d_sub + 1
            sparse_meta_data["pq_ip2l2_phi"][layer_idx] = phi
        centres, _ = kmeans_keys_batched(
            source, first, n_sub, n_cent, self.kmeans_iter, book.codes, book.capacity, 0,
            tol=1e-4, seed=self.kmeans_seed + 7919 * int(layer_idx),
        )
        book.n = n_keys
        stored = centres.to(keys.dtype).reshape(B, Hkv, n_sub, n_cent, d_fit)
        sparse_meta_data["pq_centroids"][layer_idx] = stored
        # the scoring table uses the original dimensions only (pq_top_k.py:457-458); new keys are quantised
        # against the full, possibly augmented centroids
        sparse_meta_data["pq_centroids_f32"][layer_idx] = (
            stored[..., :d_sub].to(torch.float32).reshape(-1, n_cent, d_sub).contiguous())
        sparse_meta_data.setdefault("pq_centroids_fit_f32", {})[layer_idx] = (
            stored.to(torch.float32).reshape(-1, n_cent, d_fit).contiguous())
        sparse_meta_data["pq_codebook"][layer_idx] = book
        return stored, book

    def _handle_incremental_keys(self, keys: torch.Tensor, layer_idx: int, sparse_meta_data: Dict[str, Any]):
        """Later calls: quantise keys beyond init_offset + cached count with the frozen centroids."""
        B, Hkv, Lk, _ = keys.shape
        n_sub, d_sub, n_cent = self._geometry(keys)
        book: PQCodebook = sparse_meta_data["pq_codebook"][layer_idx]
        current = Lk - self.init_offset
        if current < book.n:
            raise ValueError(f"Quantized region shrunk: {current} < {book.n}")
        if current > book.n:
            n_new = current - book.n
            book.reserve(current)
            cf32 = sparse_meta_data["pq_centroids_fit_f32"][layer_idx]
            first = self.init_offset + book.n
            if self.metric == "ip":
                keys, _ = self._augmented(keys, first, n_sub, d_sub, sparse_meta_data["pq_ip2l2_phi"][layer_idx])
                first, d_sub = 0, d_sub + 1
            a = N.PqAssignArgs(
                keys.data_ptr(), keys.stride(0), keys.stride(1), keys.stride(2), N.dtype_code(keys.dtype),
                B, Hkv, n_sub, d_sub, n_cent, first, n_new,
                cf32.data_ptr(), book.codes.data_ptr(), book.capacity, book.n,
                None, None, 1, None, N.stream_ptr(keys.device),
            )
            N.call("sah_pq_kmeans_assign", a)
            book.n = current
        return sparse_meta_data["pq_centroids"][layer_idx], book

    def add_mask(self, keys, queries, values, attention_mask, scaling, dropout, sparse_meta_data,
                 previous_mask: Mask, **kwargs: Dict[str, Any]) -> Mask:
        layer_idx = self._validate_inputs(sparse_meta_data, kwargs)
        if previous_mask.is_full_mask():
            return previous_mask
        dims = self._extract_tensor_dimensions(keys, queries)
        k_eff = self._calculate_effective_size(self.heavy_size, dims.seq_len_keys)
        if self._should_use_full_attention(dims, k_eff):
            return self._create_full_mask(dims, previous_mask.dtype, previous_mask.device)
        N.require_device(keys, "keys")
        N.require_device(queries, "queries")
        _get_num_key_value_groups(queries, keys)
        q = _inner_contiguous(queries)
        k = _inner_contiguous(keys)
        self._initialize_pq_cache(sparse_meta_data, layer_idx)
        if sparse_meta_data["pq_centroids"][layer_idx] is None:
            _, book = self._perform_kmeans_clustering(k, layer_idx, sparse_meta_data)
        else:
            _, book = self._handle_incremental_keys(k, layer_idx, sparse_meta_data)

        B, Hq, Lq, _ = q.shape
        Hkv = k.shape[1]
        n_sub, d_sub, n_cent = self._geometry(k)
        n_cand = book.n
        rows = previous_mask.to_rows(extra=k_eff)
        keybuf = score_key_buffer(rows.n_rows, n_cand, q.dtype, q.device)
        cf32 = sparse_meta_data["pq_centroids_f32"][layer_idx]
        lut = adc_lut_buffer(B, Hq, Hkv, Lq, n_sub, n_cent, q.dtype, q.device)
        a = N.PqAdcArgs(
            q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), N.dtype_code(q.dtype),
            B, Hq, Hkv, Lq, n_sub, d_sub, n_cent,
            cf32.data_ptr(), book.codes.data_ptr(), book.capacity, n_cand,
            keybuf.data_ptr(), keybuf.stride(0), lut.data_ptr(), lut.numel(), N.stream_ptr(q.device),
        )
        stored = sparse_meta_data["pq_centroids"][layer_idx]
        if stored.dtype == q.dtype and stored.dtype != torch.float32 and stored.shape[-1] == d_sub and stored.is_contiguous():
            a.centres_narrow = stored.data_ptr()   # the table is built from the 16-bit centroids: half the bytes
        N.call("sah_pq_adc_scores", a)
        excluded = sortable_key_of(torch.finfo(q.dtype).min, q.dtype)
        self._select_into_rows(rows, keybuf, 32 if q.dtype == torch.float32 else 16, n_cand, self.init_offset, k_eff, excluded)
        return Mask.create_mask_from_rows(self._mask_shape(dims), rows, previous_mask.dtype)

    @classmethod
    def create_from_config(cls, config: MaskerConfig) -> "PQCache":
        if not isinstance(config, PQCacheConfig):
            raise ValueError(f"Invalid config type: {type(config)}")
        return cls(config)
