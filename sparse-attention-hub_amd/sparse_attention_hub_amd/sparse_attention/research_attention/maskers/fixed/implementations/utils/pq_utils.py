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

from typing import Optional, Tuple

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


def ip2l2_augment(xb: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Append sqrt(phi - ||x||^2), phi = max squared norm per group (pq_utils.py:585-612)."""
    norms_sq = (xb ** 2).sum(dim=2, keepdim=True)
    phi = norms_sq.max(dim=1, keepdim=True)[0]
    return torch.cat([xb, torch.sqrt(phi - norms_sq)], dim=2), phi


def ip2l2_augment_queries(xq: torch.Tensor, phi: torch.Tensor) -> torch.Tensor:
    """Append a zero column (pq_utils.py:615-640)."""
    zero = torch.zeros(xq.shape[0], xq.shape[1], 1, dtype=xq.dtype, device=xq.device)
    return torch.cat([xq, zero], dim=2)
