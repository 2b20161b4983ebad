"""CPU oracle of the ResearchAttention decode path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain torch-CPU ops and in the reference's own op order
and dtypes, what skylight-org/sparse-attention-hub computes on this path: dense
(B, Hq, Lq, Lk) weight masks, `repeat_kv`, scores in the query dtype, full-key fp32
softmax with inverse mask weights. Only `tests/`, `__graft_entry__.smoke()` and
the `cpu_baseline` leg of `bench.py` may import it, and only as the checker or as
the timed CPU baseline; nothing under `sparse-attention-hub_amd/` does.

Every function cites the reference lines it follows (paths relative to the
reference checkout, `sparse_attention_hub/sparse_attention/...`).

One deliberate difference, stated once: where the reference calls `torch.topk`
(whose choice among equal scores is unspecified and pinned by none of its tests)
the oracle takes a stable descending sort, i.e. ties go to the lowest key index.
That is the canonical rule the kernels implement; parity with `torch.topk` itself
is tie-aware (same keys strictly above the k-th score, same count at it).

Pinning (tests/test_oracle_golden.py, tests/test_oracle_adaptive.py): every function below has a
check that a dropped term, a wrong sign or index or a transposed operand fails.
* From the reference's own unit tests: Sink/Local patterns and full-mask shortcuts, Mask
  index/ptr vectors, merge known answers, top-k known answers and invariants, pairwise distances,
  two-blob recovery, ip->l2 augmentation, ADC manual check, PQ full-attention rule, adaptive range /
  base count / failure-rate bar, sink-logit closed form, HF eager attention equality.
* Where the reference holds no vector, from what the mathematics fixes: `hash_signatures` against
  per-head `torch.nn.functional.linear` layers; `hash_topk`'s selected set against a column-by-column
  sort by (-score, column) over the inactive columns; `pq_split` / `pq_split_ip` against explicit
  (batch, head, sub-space) loops; `kmeans_lloyd` by hand-computed Lloyd steps including the
  empty-cluster reseed; `adaptive_exp_scores` against an fp64 evaluation of the definition;
  `adaptive_budget` against hand arithmetic; Philox4x32-10 against the published known-answer vectors;
  `research_attention` (the chain) by composing the pieces on a brute-forceable size; the training-mode dropout of
  `masked_attention` against the definition of `torch.nn.functional.dropout` in fp64 and single Philox calls.
Not reproducible by any restatement, because the reference leaves them to torch's RNG or to an
unspecified library choice: which samples `torch.randint` draws (adaptive / random sampling, k-means
initialisation and reseeding; the oracle takes the draws or the start centres as inputs, or draws
with Philox), which elements `torch.nn.functional.dropout` zeroes in training mode (Philox here as well) and which of several equal scores `torch.topk` keeps (lowest index here).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from statistics import NormalDist
from typing import Callable, Dict, List, Optional, Sequence, Tuple, Union

import torch

Size = Union[int, float]


# --------------------------------------------------------------------------- masks
@dataclass
class OMask:
    """'empty' | 'full' | 'dense' (weights (B, Hq, Lq, Lk) in `dtype`)."""

    kind: str
    shape: Tuple[int, int, int, int]
    dtype: torch.dtype
    dense: Optional[torch.Tensor] = None

    @staticmethod
    def empty(shape, dtype) -> "OMask":
        return OMask("empty", tuple(shape), dtype)

    @staticmethod
    def full(shape, dtype) -> "OMask":
        return OMask("full", tuple(shape), dtype)

    def to_dense(self) -> torch.Tensor:
        # utils/mask.py:577-611
        if self.kind == "full":
            return torch.ones(self.shape, dtype=self.dtype)
        if self.kind == "empty":
            return torch.zeros(self.shape, dtype=self.dtype)
        return self.dense

    def index_form(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """flat int64 indices (row * Lk + col, ascending), ptr, data — utils/mask.py:510-575."""
        d = self.to_dense()
        n_rows = d.numel() // d.shape[-1]
        flat = d.reshape(-1)
        idx = torch.nonzero(flat, as_tuple=False).squeeze(-1)
        cnt = torch.count_nonzero(d.reshape(n_rows, -1), dim=1)
        ptr = torch.cat([torch.zeros(1, dtype=torch.long), torch.cumsum(cnt, 0)])
        return idx, ptr, flat[idx]


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """utils/kv_utils.py:5-20: query head h reads kv head h // n_rep."""
    return x if n_rep == 1 else torch.repeat_interleave(x, n_rep, dim=1)


def effective_size(size: Size, n_keys: int) -> int:
    """maskers/base.py:152-158."""
    return int(size * n_keys) if isinstance(size, float) else int(size)


def merge_dense(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """utils/mask.py:875-877."""
    return torch.clamp(a + b, 0.0, 1.0)


def stable_topk(scores: torch.Tensor, k: int) -> torch.Tensor:
    """k best per row, equal scores resolved to the lowest index (see module docstring)."""
    return torch.argsort(scores, dim=-1, descending=True, stable=True)[..., :k]


# ------------------------------------------------------------------- sink / local
def sink(prev: OMask, sink_size: Size) -> OMask:
    """SinkMasker.add_mask — basic_fixed.py:384-428, :354-363."""
    if prev.kind == "full":
        return prev
    Lk = prev.shape[-1]
    s = effective_size(sink_size, Lk)
    if Lk <= s:
        return OMask.full(prev.shape, prev.dtype)
    d = prev.to_dense().clone()
    d[..., :s] = 1.0
    return OMask("dense", prev.shape, prev.dtype, d)


def local(prev: OMask, window_size: Size) -> OMask:
    """LocalMasker.add_mask / update_core — basic_fixed.py:180-224, :48-67."""
    if prev.kind == "full":
        return prev
    _, _, Lq, Lk = prev.shape
    w = effective_size(window_size, Lk)
    if Lk <= w + Lq:
        return OMask.full(prev.shape, prev.dtype)
    d = prev.to_dense().clone()
    for qi in range(Lq):
        last = Lk - Lq + qi
        d[..., qi, last - w + 1 : last + 1] = 1.0
        d[..., qi, last + 1 :] = 0.0  # future positions are cleared, whoever set them
    return OMask("dense", prev.shape, prev.dtype, d)


# -------------------------------------------------------------------- oracle top-k
def qk_scores(q: torch.Tensor, k: torch.Tensor, attention_mask: Optional[torch.Tensor]) -> torch.Tensor:
    """Un-scaled scores in the query dtype — oracle_top_k.py:70-72."""
    kk = repeat_kv(k, q.shape[1] // k.shape[1])
    s = torch.matmul(q, kk.transpose(-2, -1))
    if attention_mask is not None:
        s = s + attention_mask[:, :, :, : kk.shape[-2]]
    return s


def oracle_topk(prev: OMask, q: torch.Tensor, k: torch.Tensor, attention_mask: Optional[torch.Tensor],
                heavy_size: Size) -> OMask:
    """OracleTopK.add_mask — oracle_top_k.py:172-218, :48-80, :102-125."""
    if prev.kind == "full":
        return prev
    Lk = prev.shape[-1]
    kk = effective_size(heavy_size, Lk)
    if Lk <= kk:
        return OMask.full(prev.shape, prev.dtype)
    d = prev.to_dense().clone()
    s = qk_scores(q, k, attention_mask).clone()
    s[d != 0] = torch.finfo(prev.dtype).min
    idx = stable_topk(s, kk)
    d.scatter_(-1, idx, 1.0)
    return OMask("dense", prev.shape, prev.dtype, d)


# ------------------------------------------------------------------ hash attention
_ACT: Dict[str, Callable[[torch.Tensor], torch.Tensor]] = {
    "relu": torch.nn.functional.relu,
    "silu": torch.nn.functional.silu,
    "gelu": torch.nn.functional.gelu,
    "tanh": torch.tanh,
}


def hash_signatures(x: torch.Tensor, matrices: Sequence[torch.Tensor], biases: Sequence[torch.Tensor],
                    activation: str) -> torch.Tensor:
    """+-1 (0 at exact zero) signatures (B, H, L, bits) — hashattention_top_k.py:203-253."""
    act = _ACT[activation]
    y = x
    for i in range(len(matrices) - 1):
        y = torch.einsum("bhsd,hde->bhse", y, matrices[i]) + biases[i].unsqueeze(0).unsqueeze(2)
        y = act(y)
    if len(matrices) > 0:
        y = torch.einsum("bhsd,hde->bhse", y, matrices[-1]) + biases[-1].unsqueeze(0).unsqueeze(2)
    return torch.sign(y)


def pack_signatures(sig: torch.Tensor) -> torch.Tensor:
    """int64 (..., 2): plane 0 bit e = (sig[..., e] > 0), plane 1 bit e = (sig[..., e] != 0),
    LSB first (the kernels' packing of a {-1, 0, +1} signature)."""
    shifts = torch.arange(sig.shape[-1], dtype=torch.int64)
    pos = ((sig > 0).to(torch.int64) << shifts).sum(-1)
    nonzero = ((sig != 0).to(torch.int64) << shifts).sum(-1)
    return torch.stack([pos, nonzero], dim=-1)


def _popcount64(x: torch.Tensor) -> torch.Tensor:
    pop = torch.zeros_like(x)
    for b in range(32):
        pop += (x >> b) & 1
    return pop


def signature_scores_from_codes(qcodes: torch.Tensor, kcodes: torch.Tensor) -> torch.Tensor:
    """q_sig @ k_sig^T from packed planes: popcount(nz) - 2 popcount((q ^ k) & nz), nz = both
    non-zero. qcodes (..., Lq, 2), kcodes (..., Lk, 2) -> (..., Lq, Lk). Closed form; equals
    bits - 2 * Hamming when no entry is zero."""
    nz = qcodes[..., 1].unsqueeze(-1) & kcodes[..., 1].unsqueeze(-2)
    diff = (qcodes[..., 0].unsqueeze(-1) ^ kcodes[..., 0].unsqueeze(-2)) & nz
    return _popcount64(nz) - 2 * _popcount64(diff)


def hash_topk(prev: OMask, q: torch.Tensor, k: torch.Tensor, attention_mask: Optional[torch.Tensor],
              heavy_size: Size, weights: Dict[str, List[torch.Tensor]], activation: str,
              key_signatures: Optional[torch.Tensor] = None,
              query_signatures: Optional[torch.Tensor] = None) -> Tuple[OMask, torch.Tensor]:
    """HashAttentionTopKMasker.add_mask — hashattention_top_k.py:79-127, :343-371; top-k on
    inactive positions — fixed/base.py:74-85. `key_signatures` plays the role of the per-layer
    cache (:255-341): given, only keys beyond its length are hashed. `query_signatures`, when
    given, replaces the query MLP (used to test selection separately from MLP rounding).
    Returns (mask, key signatures)."""
    G = q.shape[1] // k.shape[1]
    kk = repeat_kv(k, G)
    if key_signatures is None:
        ksig = hash_signatures(kk, weights["key_matrix"], weights["key_bias"], activation)
    else:
        n_old = key_signatures.shape[2]
        if kk.shape[2] < n_old:
            raise ValueError("key count shrank")
        ksig = key_signatures
        if kk.shape[2] > n_old:
            new = hash_signatures(kk[:, :, n_old:, :], weights["key_matrix"], weights["key_bias"], activation)
            ksig = torch.cat([key_signatures, new], dim=2)
    if prev.kind == "full":
        return prev, ksig
    Lk = prev.shape[-1]
    kcount = effective_size(heavy_size, Lk)
    if Lk <= kcount:
        return OMask.full(prev.shape, prev.dtype), ksig
    qsig = query_signatures
    if qsig is None:
        qsig = hash_signatures(q, weights["query_matrix"], weights["query_bias"], activation)
    s = torch.matmul(qsig.to(ksig.dtype), ksig.transpose(-2, -1))
    if attention_mask is not None:
        s = s + attention_mask[:, :, :, :Lk]
    d = prev.to_dense()
    s = s.clone()
    s[d != 0] = float("-inf")
    idx = stable_topk(s, kcount)
    new_mask = torch.zeros(prev.shape, dtype=prev.dtype)
    new_mask.scatter_(-1, idx, torch.ones_like(idx, dtype=prev.dtype))
    if prev.kind == "empty":
        return OMask("dense", prev.shape, prev.dtype, new_mask), ksig
    return OMask("dense", prev.shape, prev.dtype, merge_dense(d, new_mask)), ksig


# ------------------------------------------------------------------------- PQCache
def pairwise_sq_dist(x: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    """(b, n, k) squared distances — pq_utils.py:220-257."""
    return ((x.unsqueeze(2) - c.unsqueeze(1)) ** 2.0).sum(dim=-1)


def kmeans_lloyd(X: torch.Tensor, centres: torch.Tensor, iter_limit: int, tol: float = 1e-4,
                 reseed_idx: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """kmeans_batched given initial centres — pq_utils.py:260-438. X (b, n, d), centres (b, k, d).
    Returns (codes of the assignment that preceded the last centre update, centres in X's dtype).
    Empty clusters take X[g, reseed_idx[it, g, c]] (the reference draws these with torch.randint)."""
    out_dtype = X.dtype
    X = X.float()
    state = centres.float().clone()
    b, n, _ = X.shape
    kc = state.shape[1]
    it = 0
    while True:
        codes = torch.argmin(pairwise_sq_dist(X, state), dim=2)
        prev = state.clone()
        onehot = torch.nn.functional.one_hot(codes, kc).float()
        sums = (X.unsqueeze(2) * onehot.unsqueeze(-1)).sum(dim=1)
        counts = onehot.sum(dim=1)
        new = sums / counts.clamp(min=1).unsqueeze(-1)
        empty = counts == 0
        if empty.any():
            if reseed_idx is None:
                raise ValueError("empty cluster and no reseed indices given")
            pick = X[torch.arange(b).unsqueeze(1), reseed_idx[it].long()]
            new = torch.where(empty.unsqueeze(-1), pick, new)
        state = new
        shift = torch.sqrt(((state - prev) ** 2).sum(dim=2)).sum(dim=1)
        it += 1
        if (shift ** 2 < tol).all():
            break
        if iter_limit != 0 and it >= iter_limit:
            break
    return codes, state.to(out_dtype)


def pq_split(keys: torch.Tensor, init_offset: int, n_sub: int) -> torch.Tensor:
    """(B*Hkv*n_sub, n, d_sub) view of keys[:, :, init_offset:] — pq_top_k.py:216-231."""
    B, H, L, D = keys.shape
    d = D // n_sub
    kc = keys[:, :, init_offset:, :]
    return kc.reshape(B, H, L - init_offset, n_sub, d).transpose(2, 3).reshape(-1, L - init_offset, d)


def ip2l2_augment(xb: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(n_groups, n, d) -> (n_groups, n, d + 1) with the extra column sqrt(phi - ||x||^2),
    phi = largest squared norm of the group; phi (n_groups, 1, 1) — pq_utils.py:585-612."""
    norms_sq = (xb ** 2).sum(dim=2, keepdim=True)
    phi = norms_sq.max(dim=1, keepdim=True)[0]
    return torch.cat([xb, torch.sqrt(phi - norms_sq)], dim=2), phi


def ip2l2_augment_queries(xq: torch.Tensor) -> torch.Tensor:
    """Queries (and keys quantised later) get a zero column — pq_utils.py:615-640."""
    return torch.cat([xq, torch.zeros(xq.shape[0], xq.shape[1], 1, dtype=xq.dtype)], dim=2)


def pq_split_ip(keys: torch.Tensor, init_offset: int, n_sub: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """The vectors metric="ip" clusters: sub-vectors of keys[:, :, init_offset:] per (b, kv head,
    sub-space) group, augmented in the key dtype — pq_top_k.py:219-236. Returns (X, phi)."""
    B, H, Lk, D = keys.shape
    d = D // n_sub
    flat = keys[:, :, init_offset:, :].reshape(B, H, Lk - init_offset, n_sub, d).transpose(2, 3).reshape(-1, Lk - init_offset, d)
    return ip2l2_augment(flat)


def pq_quantize_new(new_keys: torch.Tensor, centroids: torch.Tensor) -> torch.Tensor:
    """codes (B, n_new, Hkv, n_sub) in the key dtype's arithmetic — pq_top_k.py:343-404. Centroids one
    dimension wider than the sub-vectors are those of metric="ip": the new keys then get a zero column."""
    B, H, n_new, D = new_keys.shape
    n_sub = centroids.shape[2]
    d = D // n_sub
    nk = new_keys.reshape(B, H, n_new, n_sub, d).transpose(2, 3)
    if centroids.shape[-1] == d + 1:
        nk = ip2l2_augment_queries(nk.reshape(-1, n_new, d)).reshape(B, H, n_sub, n_new, d + 1)
    dist = torch.sum((nk.unsqueeze(4) - centroids.unsqueeze(3)) ** 2, dim=-1)
    return torch.argmin(dist, dim=-1).permute(0, 3, 1, 2)


def pq_scores(q: torch.Tensor, n_kv_heads: int, centroids: torch.Tensor, codebook: torch.Tensor) -> torch.Tensor:
    """ADC scores (B, Hq, Lq, n) in the query dtype — pq_top_k.py:406-490.
    centroids (B, Hkv, n_sub, k, d[+1]); codebook int64 (B, n, Hkv, n_sub)."""
    B, Hq, Lq, D = q.shape
    n_sub = codebook.shape[3]
    d = D // n_sub
    G = Hq // n_kv_heads
    qt = q.reshape(B, Hq, Lq, n_sub, d).transpose(2, 3)
    cent = torch.repeat_interleave(centroids, G, dim=1)[..., :d].transpose(3, 4)
    table = torch.matmul(qt, cent)  # (B, Hq, n_sub, Lq, k)
    codes = repeat_kv(codebook.permute(0, 2, 3, 1), G).unsqueeze(3).expand(-1, -1, -1, Lq, -1)
    return torch.gather(table, 4, codes).sum(dim=2)


def pq_topk(prev: OMask, scores: torch.Tensor, heavy_size: Size, init_offset: int) -> OMask:
    """_create_pq_mask + merge — pq_top_k.py:492-537, :150."""
    Lk = prev.shape[-1]
    kk = effective_size(heavy_size, Lk)
    d = prev.to_dense()
    s = scores.clone()
    s[d[..., init_offset : init_offset + scores.shape[3]] != 0] = torch.finfo(scores.dtype).min
    idx = stable_topk(s, kk) + init_offset
    new_mask = torch.zeros(prev.shape, dtype=prev.dtype)
    new_mask.scatter_(-1, idx, torch.ones_like(idx, dtype=prev.dtype))
    if prev.kind == "empty":
        return OMask("dense", prev.shape, prev.dtype, new_mask)
    return OMask("dense", prev.shape, prev.dtype, merge_dense(d, new_mask))


def pq_should_use_full(n_keys: int, n_queries: int, heavy: int, init_offset: int, pq_bits: int) -> bool:
    """pq_top_k.py:167-174."""
    return n_keys <= heavy + init_offset + n_queries + 2 ** pq_bits


# ------------------------------------------------------------- adaptive sampling
def adaptive_exp_scores(q, k, scaling: float, attention_mask) -> torch.Tensor:
    """exp(q k^T * scaling + mask - rowmax) in the query dtype — adaptive_sampling.py:183-197."""
    kk = repeat_kv(k, q.shape[1] // k.shape[1])
    raw = torch.matmul(q, kk.transpose(-2, -1)) * scaling
    if attention_mask is not None:
        raw = raw + attention_mask[:, :, :, : kk.shape[-2]]
    return torch.exp(raw - torch.max(raw, dim=-1, keepdim=True)[0])


def apply_inv_mask_dense(x: torch.Tensor, mask_dense: torch.Tensor) -> torch.Tensor:
    """utils/mask.py:718-740."""
    return x * (1.0 / (mask_dense + 1e-6) * (mask_dense != 0))


def adaptive_sampling_range(n_keys: int, init_offset: Size, local_offset: Size) -> Tuple[int, int, int]:
    """adaptive_sampling.py:203-228."""
    start = int(init_offset * n_keys) if isinstance(init_offset, float) else init_offset
    end = n_keys - (int(local_offset * n_keys) if isinstance(local_offset, float) else local_offset)
    return start, end, end - start


def adaptive_base_count(rate: Size, sampling_range: int) -> int:
    """adaptive_sampling.py:230-235."""
    return max(2, rate) if isinstance(rate, int) else max(2, int(rate * sampling_range))


def adaptive_budget_formula(std: torch.Tensor, est_den: torch.Tensor, n: int, epsilon: float, ppf: float) -> torch.Tensor:
    """_compute_adaptive_budget — adaptive_sampling.py:282-302 (int64, before the base-count clamp)."""
    err = torch.clamp(epsilon * est_den, min=1e-8)
    return torch.clamp((ppf * std * n / err) ** 2, min=1.0, max=float(n)).long()


def adaptive_budget(prev: OMask, expw: torch.Tensor, base_idx: torch.Tensor, start: int, end: int,
                    epsilon: float, delta: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """(budget int64 (B,H,Lq,1), probability in the mask dtype) from given base draws
    `base_idx` (B,H,Lq,nb) — adaptive_sampling.py:237-302, :365-397."""
    n = end - start
    nb = base_idx.shape[-1]
    ppf = float(NormalDist().inv_cdf(1 - delta))
    if prev.kind in ("empty", "full"):
        static_den = expw.sum(dim=-1, keepdim=True)
    else:
        static_den = apply_inv_mask_dense(expw, prev.to_dense()).sum(dim=-1, keepdim=True)
    vals = torch.gather(expw, -1, base_idx)
    std = torch.clamp(torch.std(vals.reshape(-1, nb), dim=-1, keepdim=True), min=1e-8).view(*expw.shape[:3], 1)
    base_dense = torch.zeros(prev.shape, dtype=prev.dtype)
    base_dense.scatter_(-1, base_idx, torch.full_like(base_idx, nb / n, dtype=expw.dtype).to(prev.dtype))
    sampled_den = apply_inv_mask_dense(expw, base_dense).sum(dim=-1, keepdim=True)
    est = static_den + sampled_den
    budget = adaptive_budget_formula(std, est, n, epsilon, ppf)
    budget = torch.clamp(budget, min=nb, max=n)
    return budget, (budget / n).to(prev.dtype)


def adaptive_merge(prev: OMask, draws: List[torch.Tensor], prob: torch.Tensor) -> OMask:
    """Merge rows of sampled columns (`draws[r]` for row r, with replacement) carrying weight
    prob[r] into prev: duplicates collapse, clamp(prev + p) — mask_attention_utils.py:105-184,
    utils/mask.py:595-609, :875-877."""
    n_rows = len(draws)
    Lk = prev.shape[-1]
    samp = torch.zeros((n_rows, Lk), dtype=prev.dtype)
    p = prob.reshape(-1)
    for r in range(n_rows):
        samp[r, draws[r].long()] = p[r]
    samp = samp.view(prev.shape)
    if prev.kind == "empty":
        return OMask("dense", prev.shape, prev.dtype, samp)
    return OMask("dense", prev.shape, prev.dtype, merge_dense(prev.to_dense(), samp))


# Counter-based random numbers for the sampling masker. The reference draws with
# torch.randint from torch's global generator (adaptive_sampling.py:251-256,
# utils/mask_attention_utils.py:152-158); its streams are generator- and
# device-specific, so only their distribution (uniform on [start, end), with
# replacement) is part of the contract. The kernels use Philox4x32-10 (Salmon, Moraes,
# Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11); this is the same
# published algorithm in numpy, pinned in the tests by the paper's known-answer vectors.
_PHILOX_M0 = 0xD2511F53
_PHILOX_M1 = 0xCD9E8D57
_PHILOX_W0 = 0x9E3779B9
_PHILOX_W1 = 0xBB67AE85


def philox4x32_10(counter, key):
    """counter: (..., 4) uint32, key: (2,) uint32 -> (..., 4) uint32."""
    import numpy as np

    c = np.asarray(counter, dtype=np.uint64) & 0xFFFFFFFF
    c0, c1, c2, c3 = (c[..., i].copy() for i in range(4))
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = c0 * _PHILOX_M0
        p1 = c2 * _PHILOX_M1
        n0 = (p1 >> 32) ^ c1 ^ k0
        n2 = (p0 >> 32) ^ c3 ^ k1
        c0, c1, c2, c3 = n0, p1 & 0xFFFFFFFF, n2, p0 & 0xFFFFFFFF
        k0 = (k0 + _PHILOX_W0) & 0xFFFFFFFF
        k1 = (k1 + _PHILOX_W1) & 0xFFFFFFFF
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def philox_columns(seed: int, offset: int, row: int, n: int, start: int, rng: int) -> torch.Tensor:
    """Draws 0..n-1 of mask row `row`: draw i is word i % 4 of the block with counter
    (i // 4, row, offset lo, offset hi) under key (seed lo, seed hi), mapped to the column
    start + ((u * range) >> 32)."""
    import numpy as np

    n_blocks = (n + 3) // 4
    ctr = np.zeros((n_blocks, 4), dtype=np.uint64)
    ctr[:, 0] = np.arange(n_blocks, dtype=np.uint64)
    ctr[:, 1] = row
    ctr[:, 2] = offset & 0xFFFFFFFF
    ctr[:, 3] = (offset >> 32) & 0xFFFFFFFF
    u = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)).reshape(-1)[:n].astype(np.uint64)
    cols = start + ((u * np.uint64(rng)) >> np.uint64(32)).astype(np.int64)
    return torch.from_numpy(cols)


def adaptive_sampling(prev: OMask, q, k, attention_mask, scaling: float, rate: Size, epsilon: float, delta: float,
                      init_offset: Size, local_offset: Size, seed: int, offset: int,
                      budget_override: Optional[torch.Tensor] = None):
    """AdaptiveSamplingMasker.add_mask — adaptive_sampling.py:304-407, with the draws of
    call `offset` taken from Philox (base sample: offset, budgeted sample: offset + 1).
    `budget_override` (int64, one per row) replaces the computed budget, so that the merge
    can be checked bit-exactly for a budget obtained elsewhere. Returns (mask, budget, prob)."""
    if prev.kind == "full":
        return prev, None, None
    if rate == 0:
        return prev, None, None
    B, H, Lq, Lk = prev.shape
    start, end, n = adaptive_sampling_range(Lk, init_offset, local_offset)
    if n < 2:
        return OMask.full(prev.shape, prev.dtype), None, None
    expw = adaptive_exp_scores(q, k, scaling, attention_mask)
    nb = adaptive_base_count(rate, n)
    R = B * H * Lq
    base = torch.stack([philox_columns(seed, offset, r, nb, start, n) for r in range(R)]).view(B, H, Lq, nb)
    budget, prob = adaptive_budget(prev, expw, base, start, end, epsilon, delta)
    if budget_override is not None:
        budget = budget_override.view(B, H, Lq, 1).to(torch.int64)
        prob = (budget / n).to(prev.dtype)
    flat = budget.reshape(-1)
    draws = [philox_columns(seed, offset + 1, r, int(flat[r]), start, n) for r in range(R)]
    return adaptive_merge(prev, draws, prob), budget, prob


def random_sampling(prev: OMask, rate: float, seed: int, offset: int) -> OMask:
    """RandomSamplingMasker.add_mask — random_sampling.py:95-193: int(rate * n_keys) uniform draws per row on
    [0, n_keys) with replacement (here: Philox call `offset`), weight `rate` in the mask dtype, dense merge."""
    if prev.kind == "full":
        return prev
    B, H, Lq, Lk = prev.shape
    n = int(rate * Lk)
    R = B * H * Lq
    draws = [philox_columns(seed, offset, r, n, 0, Lk) for r in range(R)]
    prob = torch.full((R,), rate, dtype=prev.dtype)
    return adaptive_merge(prev, draws, prob)


# ----------------------------------------------------------------------- attention
def dropout_keep(seed: int, offset: int, n_rows: int, n_keys: int, p: float) -> torch.Tensor:
    """(n_rows, n_keys) bool: entry (r, j) survives a dropout of probability p when word 0 of
    Philox4x32-10(counter (j, r, offset lo, offset hi), key (seed lo, seed hi)) is at least p * 2^32."""
    import numpy as np

    ctr = np.zeros((n_rows, n_keys, 4), dtype=np.uint64)
    ctr[:, :, 0] = np.arange(n_keys, dtype=np.uint64)[None, :]
    ctr[:, :, 1] = np.arange(n_rows, dtype=np.uint64)[:, None]
    ctr[:, :, 2] = offset & 0xFFFFFFFF
    ctr[:, :, 3] = (offset >> 32) & 0xFFFFFFFF
    u = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))[..., 0].astype(np.uint64)
    thresh = max(1, min(0xFFFFFFFF, int(np.float64(np.float32(p)) * 4294967296.0)))
    return torch.from_numpy(u >= np.uint64(thresh))


def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attention_mask: Optional[torch.Tensor],
                     sinks: Optional[torch.Tensor], scaling: float, mask: OMask,
                     accumulate: torch.dtype = torch.float32,
                     dropout: Optional[Tuple[float, int, int]] = None,
                     dropout_numerator_only: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """(out (B, Lq, Hq, D), weights (B, Hq, Lq, Lk)) in the query dtype —
    mask_attention_utils.py:187-240 (exp weights), :357-402 (sink logit), :406-491 (num/den).
    `accumulate=torch.float64` gives a high-precision variant for tolerance studies.
    `dropout` = (p, seed, offset): training-mode dropout of the exp weights (:234-238, torch.nn.functional.dropout:
    an element is zeroed with probability p, the others are scaled by 1 / (1 - p)), with the element's fate drawn
    from Philox (dropout_keep) instead of torch's generator. `dropout_numerator_only`: the dropped entries stay in the
    denominator - dropout of the normalised probabilities, what scaled_dot_product_attention(dropout_p=...) does on the
    reference's dense path (:40-52)."""
    G = q.shape[1] // k.shape[1]
    kk = repeat_kv(k, G).to(accumulate)
    vv = repeat_kv(v, G).to(accumulate)
    logits = torch.matmul(q.to(accumulate), kk.transpose(2, 3)) * scaling
    if attention_mask is not None:
        logits = logits + attention_mask[:, :, :, : kk.shape[-2]].to(accumulate)
    old_max = torch.max(logits, dim=-1, keepdim=True)[0]
    e = torch.exp(logits - old_max)
    if mask.kind == "dense":
        e = apply_inv_mask_dense(e, mask.dense)
    if dropout is not None and dropout[0] > 0.0:
        p, seed, offset = dropout
        B, H, Q, Lk = e.shape
        keep = dropout_keep(seed, offset, B * H * Q, Lk, p).view(B, H, Q, Lk)
        den_e = e
        e = e * keep.to(accumulate) * (1.0 / (1.0 - float(torch.tensor(p, dtype=torch.float32))))
        if not dropout_numerator_only:
            den_e = e
    else:
        den_e = e
    num = torch.matmul(e, vv)
    den = den_e.sum(dim=-1, keepdim=True)
    if sinks is not None:
        B, H, Q = q.shape[0], q.shape[1], q.shape[2]
        srow = sinks.view(1, H, 1, 1).expand(B, H, Q, 1).to(accumulate)
        new_max = torch.maximum(old_max, srow)
        scale = torch.exp(old_max - new_max)
        num, den, e = num * scale, den * scale, e * scale
        den = den + torch.exp(srow - new_max)
    out = (num / den).to(q.dtype).transpose(1, 2).contiguous()
    return out, (e / den).to(q.dtype)


# --------------------------------------------------------------- chain composition
def research_attention(masker_specs: Sequence[Tuple], q, k, v, attention_mask, scaling: float,
                       sinks: Optional[torch.Tensor] = None, state: Optional[dict] = None,
                       dropout: Optional[Tuple[float, int, int]] = None):
    """ResearchAttention.custom_attention — research_attention/base.py:63-170.
    masker_specs: ("sink", size) | ("local", size) | ("oracle_topk", heavy) |
    ("hash_topk", heavy, weights, activation) | ("pq_topk", heavy, init_offset, centroids, codebook) |
    ("adaptive", rate, epsilon, delta, init_offset, local_offset, seed, offset) | ("random", rate, seed, offset).
    `dropout` = (p, seed, offset): see masked_attention. Returns (out, weights, final OMask)."""
    shape = (q.shape[0], q.shape[1], q.shape[2], k.shape[2])
    m = OMask.empty(shape, q.dtype)
    state = {} if state is None else state
    for spec in masker_specs:
        kind = spec[0]
        if kind == "sink":
            m = sink(m, spec[1])
        elif kind == "local":
            m = local(m, spec[1])
        elif kind == "oracle_topk":
            m = oracle_topk(m, q, k, attention_mask, spec[1])
        elif kind == "hash_topk":
            m, sig = hash_topk(m, q, k, attention_mask, spec[1], spec[2], spec[3], state.get("key_sig"),
                               state.get("query_sig"))
            state["key_sig"] = sig
        elif kind == "pq_topk":
            heavy, off, cent, book = spec[1], spec[2], spec[3], spec[4]
            if m.kind != "full":
                kk = effective_size(heavy, shape[-1])
                n_cent = cent.shape[3]
                if pq_should_use_full(shape[-1], shape[2], kk, off, int(math.log2(n_cent))):
                    m = OMask.full(shape, q.dtype)
                else:
                    m = pq_topk(m, pq_scores(q, k.shape[1], cent, book), heavy, off)
        elif kind == "adaptive":
            # ("adaptive", rate, epsilon, delta, init_offset, local_offset, seed, offset)
            m, budget, _ = adaptive_sampling(m, q, k, attention_mask, scaling, spec[1], spec[2], spec[3], spec[4],
                                             spec[5], spec[6], spec[7], state.get("budget"))
            state["budget_oracle"] = budget
        elif kind == "random":
            m = random_sampling(m, spec[1], spec[2], spec[3])  # ("random", rate, seed, offset)
        else:
            raise ValueError(kind)
    out, w = masked_attention(q, k, v, attention_mask, sinks, scaling, m, dropout=dropout)
    return out, w, m
