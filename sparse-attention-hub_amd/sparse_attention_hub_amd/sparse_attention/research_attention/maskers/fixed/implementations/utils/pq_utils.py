"""Batched k-means for the PQCache masker on `sah_pq_kmeans_assign` / `_update`.

Reference: maskers/fixed/implementations/utils/pq_utils.py — `kmeans_batched`
(:260-438) runs Lloyd iterations on X (b, n, d) with one-hot sums over a
materialised (b, n, k, d) tensor; `kmeans_batched_pytorch` (:547-582) wraps it.
Here the groups are the sub-spaces of the key cache itself, read in place:
group g = (batch, kv head, sub-space), vector n = keys[b, hk, key_offset + n,
s*d_sub:(s+1)*d_sub]. No (b, n, k, d) tensor exists and the loop never
synchronises with the host: convergence (all groups' squared shift < tol) sets a
device flag that turns the remaining launches into no-ops.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from ....... import _native as N


def seeded_initial_centres(n_groups: int, n_keys: int, n_cent: int, seed: int, device: torch.device) -> torch.Tensor:
    """Distinct start vectors per group: one uniform draw from each of n_cent equal strata
    of [0, n_keys). (The reference draws randperm(n)[:k] from the global RNG,
    pq_utils.py:183-217; any distinct sample is an equally valid Lloyd start.)"""
    if n_keys < n_cent:
        raise ValueError(f"k-means needs at least {n_cent} vectors, got {n_keys}")
    gen = torch.Generator(device="cpu").manual_seed(int(seed))
    u = torch.rand((n_groups, n_cent), generator=gen, dtype=torch.float64)
    edges = torch.arange(n_cent + 1, dtype=torch.float64) * (n_keys / n_cent)
    lo = edges[:-1].floor().to(torch.int64)
    hi = edges[1:].floor().to(torch.int64).clamp(max=n_keys)
    width = (hi - lo).clamp(min=1)
    idx = lo.unsqueeze(0) + (u * width.unsqueeze(0)).floor().to(torch.int64)
    return idx.clamp_(max=n_keys - 1).to(torch.int32).to(device)


def gather_sub_vectors(keys: torch.Tensor, key_offset: int, n_sub: int, idx: torch.Tensor) -> torch.Tensor:
    """fp32 [n_groups, n_idx, d_sub]: vectors idx[g, :] of every group (plumbing for the start centres)."""
    B, Hkv, _, D = keys.shape
    d_sub = D // n_sub
    idx = idx.to(torch.int64).view(B, Hkv, n_sub, -1) + key_offset
    sub = keys.reshape(B, Hkv, keys.shape[2], n_sub, d_sub)
    b_i = torch.arange(B, device=keys.device).view(B, 1, 1, 1)
    h_i = torch.arange(Hkv, device=keys.device).view(1, Hkv, 1, 1)
    s_i = torch.arange(n_sub, device=keys.device).view(1, 1, n_sub, 1)
    picked = sub[b_i, h_i, idx, s_i]  # (B, Hkv, n_sub, n_idx, d_sub)
    return picked.reshape(B * Hkv * n_sub, -1, d_sub).to(torch.float32).contiguous()


def kmeans_keys_batched(
    keys: torch.Tensor,
    key_offset: int,
    n_sub: int,
    n_cent: int,
    max_iter: int,
    codes: torch.Tensor,
    code_pitch: int,
    code_offset: int = 0,
    tol: float = 1e-4,
    cluster_centers: Optional[torch.Tensor] = None,
    seed: int = 0,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Lloyd iterations over every (batch, kv head, sub-space) group of `keys`.

    keys (B, Hkv, Lk, D) in its storage dtype; vectors key_offset.. are clustered.
    codes: uint8 buffer [B, Hkv, code_pitch, n_sub], filled at code_offset...
    Returns (centres fp32 [n_groups, n_cent, d_sub], shift2 [n_groups]). As in the
    reference the codes are the assignment against the centres that *entered* the
    last executed iteration (pq_utils.py:353 precedes :399).
    """
    N.require_device(keys, "keys")
    B, Hkv, Lk, D = keys.shape
    if D % n_sub:
        raise ValueError(f"head_dim {D} is not divisible by {n_sub} sub-spaces")
    d_sub = D // n_sub
    n_keys = Lk - key_offset
    n_groups = B * Hkv * n_sub
    dev = keys.device
    if keys.stride(-1) != 1:
        keys = keys.contiguous()
    if cluster_centers is None:
        start = seeded_initial_centres(n_groups, n_keys, n_cent, seed, dev)
        centres = gather_sub_vectors(keys, key_offset, n_sub, start)
    else:
        if tuple(cluster_centers.shape) != (n_groups, n_cent, d_sub):
            raise ValueError(
                f"cluster_centers shape mismatch. Expected ({n_groups}, {n_cent}, {d_sub}), got {tuple(cluster_centers.shape)}"
            )
        centres = cluster_centers.to(device=dev, dtype=torch.float32).contiguous().clone()
    sums = torch.empty((n_groups, n_cent, d_sub), dtype=torch.int64, device=dev)  # fixed point: order-independent
    counts = torch.empty((n_groups, n_cent), dtype=torch.int32, device=dev)
    shift2 = torch.zeros((n_groups,), dtype=torch.float32, device=dev)
    state = torch.zeros((4,), dtype=torch.int32, device=dev)
    gen = torch.Generator(device="cpu").manual_seed(int(seed) + 1)
    reseed = torch.randint(0, n_keys, (max(max_iter, 1), n_groups, n_cent), generator=gen, dtype=torch.int32).to(dev)
    dt = N.dtype_code(keys.dtype)
    stream = N.stream_ptr(dev)
    absmax = torch.zeros((1,), dtype=torch.int32, device=dev)
    N.call("sah_pq_keys_absmax", N.PqAbsmaxArgs(
        keys.data_ptr(), keys.stride(0), keys.stride(1), keys.stride(2), dt, B, Hkv, n_sub * d_sub, key_offset, n_keys,
        absmax.data_ptr(), stream))
    for it in range(max_iter):
        sums.zero_()
        counts.zero_()
        a = N.PqAssignArgs(
            keys.data_ptr(), keys.stride(0), keys.stride(1), keys.stride(2), dt,
            B, Hkv, n_sub, d_sub, n_cent, key_offset, n_keys,
            centres.data_ptr(), codes.data_ptr(), code_pitch, code_offset,
            sums.data_ptr(), counts.data_ptr(), 0, state[2:].data_ptr(), stream, absmax.data_ptr(),
        )
        N.call("sah_pq_kmeans_assign", a)
        u = N.PqUpdateArgs(
            keys.data_ptr(), keys.stride(0), keys.stride(1), keys.stride(2), dt,
            B, Hkv, n_sub, d_sub, n_cent, key_offset,
            centres.data_ptr(), sums.data_ptr(), counts.data_ptr(), reseed[it].data_ptr(),
            shift2.data_ptr(), float(tol), state.data_ptr(), stream, absmax.data_ptr(),
        )
        N.call("sah_pq_kmeans_update", u)
    return centres, shift2


def kmeans_batched(
    X: torch.Tensor,
    num_clusters: int,
    distance: str = "euclidean",
    cluster_centers: Optional[torch.Tensor] = None,
    tol: float = 1e-4,
    tqdm_flag: bool = False,
    iter_limit: int = 0,
    device: Optional[torch.device] = None,
    seed: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Batched k-means of X (b, n, d) under the reference's own name and argument list (pq_utils.py:260-438):
    returns (cluster choice (b, n) int64, centres (b, num_clusters, d) in X's dtype). Every group b is one
    "sub-space" of a single-head key tensor for `kmeans_keys_batched`, so the same Lloyd kernels run.

    Differences a caller can observe: codes are one byte in the kernels, so `num_clusters` is at most 256;
    `iter_limit == 0` (the reference: until convergence) runs at most 300 iterations, each a no-op once every
    group's squared centre shift has fallen below `tol`; the start is a seeded stratified sample of distinct
    vectors (`seed`, default 0) instead of torch's global RNG; `device` is ignored (X stays where it is)."""
    if X.ndim != 3:
        raise ValueError(f"Expected 3D input (b, n, d), got {X.ndim}D tensor with shape {X.shape}")
    if distance != "euclidean":
        raise NotImplementedError(
            f"Distance '{distance}' not yet implemented for batched k-means. Only 'euclidean' is supported.")
    if not 1 <= num_clusters <= 256:
        raise ValueError(f"num_clusters must be in [1, 256] (one-byte codes), got {num_clusters}")
    b, n, d = X.shape
    if d > 128 or b > 65535:
        raise ValueError(f"the Lloyd kernels cluster up to 65535 groups of vectors of at most 128 dimensions, got b={b}, d={d}")
    if cluster_centers is not None and tuple(cluster_centers.shape) != (b, num_clusters, d):
        raise ValueError(
            f"cluster_centers shape mismatch. Expected ({b}, {num_clusters}, {d}), got {tuple(cluster_centers.shape)}")
    N.require_device(X, "X")
    data = X if X.dtype in (torch.float32, torch.bfloat16, torch.float16) else X.float()
    # (b, n, d) read as keys (B = b, one kv head, n keys, head_dim d) with ONE sub-space of width d
    keys = data.contiguous().view(b, 1, n, d)
    codes = torch.empty((b, 1, n, 1), dtype=torch.uint8, device=X.device)
    centres, _ = kmeans_keys_batched(keys, 0, 1, num_clusters, iter_limit if iter_limit > 0 else 300, codes, n, 0, tol=tol,
                                     cluster_centers=cluster_centers, seed=0 if seed is None else int(seed))
    return codes.view(b, n).to(torch.int64), centres.to(X.dtype)


def kmeans_batched_pytorch(data: torch.Tensor, k: int, max_iter: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(centroids (n_groups, k, d), codes (n_groups, n_samples) int64) — the reference's wrapper
    (pq_utils.py:547-582) over `kmeans_batched`."""
    codes, centroids = kmeans_batched(X=data, num_clusters=k, distance="euclidean", cluster_centers=None, tol=1e-4,
                                      tqdm_flag=False, iter_limit=max_iter, device=data.device, seed=None)
    return centroids, codes.long()


def compute_reconstruction_errors(original_keys: torch.Tensor, centroids: torch.Tensor, codebook: torch.Tensor,
                                  pq_sub_dim: int, use_ip_metric: bool = False) -> Dict[str, float]:
    """mse / l2 / relative error of keys rebuilt from their codes (reference: pq_utils.py:643-705).
    original_keys (B, H, n, D); centroids (B, H, n_sub, n_cent, d [+1 for the ip metric]); codebook
    (B, n, H, n_sub) integer codes (the reference's layout; a `PQCodebook` is converted). A diagnostic, not on the
    decode path: one gather with torch indexing."""
    if hasattr(codebook, "to_reference"):
        codebook = codebook.to_reference()
    B, H, n, D = original_keys.shape
    n_sub = D // pq_sub_dim
    original = original_keys.transpose(1, 2).reshape(B, n, H, n_sub, pq_sub_dim)
    cents = centroids[..., :pq_sub_dim] if use_ip_metric else centroids           # (B, H, n_sub, n_cent, d)
    idx = codebook.to(torch.int64).permute(0, 2, 3, 1)                              # (B, H, n_sub, n)
    rebuilt = torch.gather(cents, 3, idx.unsqueeze(-1).expand(-1, -1, -1, -1, cents.shape[-1]))   # (B, H, n_sub, n, d)
    rebuilt = rebuilt.permute(0, 3, 1, 2, 4).to(original.dtype)
    diff = original - rebuilt
    l2 = torch.norm(diff.float()).item()
    norm = torch.norm(original.float()).item()
    return {"mse_error": torch.mean(diff.float() ** 2).item(), "l2_error": l2,
            "relative_error": l2 / norm if norm > 0 else 0.0}


def ip2l2_augment(xb: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Append sqrt(phi - ||x||^2), phi = max squared norm per group (pq_utils.py:585-612)."""
    norms_sq = (xb ** 2).sum(dim=2, keepdim=True)
    phi = norms_sq.max(dim=1, keepdim=True)[0]
    return torch.cat([xb, torch.sqrt(phi - norms_sq)], dim=2), phi


def ip2l2_augment_queries(xq: torch.Tensor, phi: torch.Tensor) -> torch.Tensor:
    """Append a zero column (pq_utils.py:615-640)."""
    zero = torch.zeros(xq.shape[0], xq.shape[1], 1, dtype=xq.dtype, device=xq.device)
    return torch.cat([xq, zero], dim=2)
