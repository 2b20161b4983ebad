"""Pins the CPU oracle (oracle/reference_path.py) before anything is compared with it.

Known answers are the ones the reference's own unit tests hold (file:line cited per
test, paths under the reference's tests/unit/sparse_attention/); what those leave
open is pinned by closed forms, library routines and brute force chosen so that a
dropped term, a wrong sign/index or a transposed operand fails.
"""
import math

import pytest
import torch

from oracle import reference_path as O


def _empty(B, H, Lq, Lk, dtype=torch.float32):
    return O.OMask.empty((B, H, Lq, Lk), dtype)


# ----------------------------------------------------------------- sink / local
def test_local_pattern_lq3_lk8_w2():
    # research_attention/maskers/fixed/implementations/test_basic_fixed.py:186-202
    m = O.local(_empty(1, 1, 3, 8), 2)
    want = torch.tensor([[0, 0, 0, 0, 1, 1, 0, 0], [0, 0, 0, 0, 0, 1, 1, 0], [0, 0, 0, 0, 0, 0, 1, 1]], dtype=torch.float32)
    assert torch.equal(m.to_dense()[0, 0], want)


def test_local_float_window_same_pattern():
    # test_basic_fixed.py:212-256: 0.25 * 8 = 2
    assert torch.equal(O.local(_empty(1, 1, 3, 8), 0.25).to_dense(), O.local(_empty(1, 1, 3, 8), 2).to_dense())


def test_local_merges_with_previous():
    # test_basic_fixed.py:299-312: previous [0,1] + local
    prev = torch.zeros(1, 1, 3, 8)
    prev[..., :2] = 1.0
    m = O.local(O.OMask("dense", (1, 1, 3, 8), torch.float32, prev), 2)
    want = torch.tensor([[1, 1, 0, 0, 1, 1, 0, 0], [1, 1, 0, 0, 0, 1, 1, 0], [1, 1, 0, 0, 0, 0, 1, 1]], dtype=torch.float32)
    assert torch.equal(m.to_dense()[0, 0], want)


def test_local_and_sink_full_shortcuts():
    # test_basic_fixed.py:71-145 (Lk <= w + Lq -> full; previous full -> full) and :433-535 (Lk <= sink -> full)
    assert O.local(_empty(1, 1, 3, 8), 5).kind == "full"       # 8 <= 5 + 3
    assert O.local(_empty(1, 1, 3, 8), 4).kind == "dense"      # 8 > 4 + 3
    assert O.local(O.OMask.full((1, 1, 3, 8), torch.float32), 2).kind == "full"
    assert O.sink(_empty(1, 1, 2, 8), 8).kind == "full"
    assert O.sink(_empty(1, 1, 2, 8), 7).kind == "dense"
    assert O.sink(O.OMask.full((1, 1, 2, 8), torch.float32), 2).kind == "full"


def test_sink_plus_previous_last_two():
    # test_basic_fixed.py (sink 4 on Lk=16 with the last two columns already active)
    prev = torch.zeros(1, 1, 1, 16)
    prev[..., -2:] = 1.0
    d = O.sink(O.OMask("dense", (1, 1, 1, 16), torch.float32, prev), 4).to_dense()[0, 0, 0]
    assert torch.equal(torch.nonzero(d).squeeze(-1), torch.tensor([0, 1, 2, 3, 14, 15]))


def test_local_clears_future_columns_set_earlier():
    # basic_fixed.py:60-66: columns beyond Lk-Lq+q are zeroed, including sink columns
    m = O.local(O.sink(_empty(1, 1, 4, 12), 10), 2)
    d = m.to_dense()[0, 0]
    assert d[0, 9] == 0 and d[0, 8] == 1      # q=0 sees up to column 8
    assert d[3, 9] == 1


def test_effective_size_truncates():
    # maskers/base.py:152-158; test_oracle_top_k.py:193-237 (0.4 * 5 = 2)
    assert O.effective_size(0.4, 5) == 2 and O.effective_size(3, 5) == 3 and O.effective_size(0.05, 32768) == 1638


# --------------------------------------------------------------------- index form
def test_index_form_known_vector():
    # utils/test_mask.py:225-252: rows [[0,2,4],[1,3,4]] of width 5 -> idx [0,2,4,6,8,9], ptr [0,3,6]
    d = torch.tensor([[1.0, 0, 0.5, 0, 0.8], [0, 0.6, 0, 0.9, 0.3]]).view(1, 1, 2, 5)
    idx, ptr, data = O.OMask("dense", (1, 1, 2, 5), torch.float32, d).index_form()
    assert idx.tolist() == [0, 2, 4, 6, 8, 9] and ptr.tolist() == [0, 3, 6]
    assert torch.allclose(data, torch.tensor([1.0, 0.5, 0.8, 0.6, 0.9, 0.3]))


def test_merge_dense_known_answer():
    # utils/test_mask.py:433-478
    a = torch.tensor([[1.0, 0.0, 0.5, 0.0, 0.0], [0.0, 0.8, 0.0, 0.0, 0.3]])
    b = torch.tensor([[0.0, 0.2, 0.5, 0.0, 0.4], [0.1, 0.0, 0.0, 0.6, 0.0]])
    assert torch.allclose(O.merge_dense(a, b), torch.tensor([[1.0, 0.2, 1.0, 0.0, 0.4], [0.1, 0.8, 0.0, 0.6, 0.3]]))


# ---------------------------------------------------------------------- top-k
def test_oracle_topk_avoids_previous_active():
    # test_oracle_top_k.py:239-305: keys 10, 5, 1, .5, .1 on channel 0, previous {0,1} -> picks {2,3}
    k = torch.zeros(1, 1, 5, 4)
    k[0, 0, :, 0] = torch.tensor([10.0, 5.0, 1.0, 0.5, 0.1])
    q = torch.zeros(1, 1, 2, 4)
    q[..., 0] = 1.0
    prev = torch.zeros(1, 1, 2, 5)
    prev[..., :2] = 1.0
    d = O.oracle_topk(O.OMask("dense", (1, 1, 2, 5), torch.float32, prev), q, k, None, 2).to_dense()
    assert torch.equal(d[0, 0, 0], torch.tensor([1.0, 1.0, 1.0, 1.0, 0.0]))
    assert torch.equal(d[0, 0, 1], torch.tensor([1.0, 1.0, 1.0, 1.0, 0.0]))


def test_stable_topk_prefers_lowest_index_and_matches_brute_force():
    s = torch.tensor([[1.0, 3.0, 3.0, 3.0, 2.0, 3.0]])
    assert O.stable_topk(s, 2).tolist() == [[1, 2]]
    g = torch.Generator().manual_seed(3)
    s = torch.randint(0, 6, (7, 40), generator=g).float()
    got = O.stable_topk(s, 9)
    for r in range(7):
        order = sorted(range(40), key=lambda j: (-s[r, j].item(), j))[:9]
        assert got[r].tolist() == order


def test_oracle_topk_counts_and_gqa_mapping():
    # test_oracle_top_k.py:147-362 invariants: exactly k new per row, none inside previous; GQA h -> h // G
    g = torch.Generator().manual_seed(0)
    q = torch.randn(2, 4, 1, 8, generator=g)
    k = torch.randn(2, 2, 50, 8, generator=g)
    prev = O.local(O.sink(_empty(2, 4, 1, 50), 3), 5)
    out = O.oracle_topk(prev, q, k, None, 7)
    new = (out.to_dense() != 0) & (prev.to_dense() == 0)
    assert torch.all(new.sum(-1) == 7)
    # brute force on one row with explicit kv-head choice
    b, h = 1, 3
    scores = torch.tensor([float(q[b, h, 0] @ k[b, h // 2, j]) for j in range(50)])
    scores[:3] = -1e30
    scores[45:] = -1e30
    want = sorted(sorted(range(50), key=lambda j: (-scores[j].item(), j))[:7])
    assert torch.nonzero(new[b, h, 0]).squeeze(-1).tolist() == want


# ---------------------------------------------------------------- hash attention
def _tiny_hat(H, D, bits, hidden, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    dims = [D, hidden, hidden, bits]
    w = {"query_matrix": [], "query_bias": [], "key_matrix": [], "key_bias": []}
    for kind in ("query", "key"):
        for i in range(3):
            w[f"{kind}_matrix"].append((torch.randn(H, dims[i], dims[i + 1], generator=g) / math.sqrt(dims[i])).to(dtype))
            w[f"{kind}_bias"].append((torch.randn(H, dims[i + 1], generator=g) / math.sqrt(dims[i])).to(dtype))
    return w


def test_hash_signatures_against_per_head_linear_layers():
    # definition hashattention_top_k.py:203-253 restated with nn.functional.linear per head (library routine)
    H, D, bits = 3, 8, 16
    w = _tiny_hat(H, D, bits, 12)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, H, 5, D, generator=g)
    sig = O.hash_signatures(x, w["key_matrix"], w["key_bias"], "silu")
    for h in range(H):
        y = x[:, h]
        for i in range(3):
            y = torch.nn.functional.linear(y, w["key_matrix"][i][h].t(), w["key_bias"][i][h])
            if i < 2:
                y = torch.nn.functional.silu(y)
        assert torch.equal(torch.sign(y), sig[:, h])
    assert sig.shape == (2, H, 5, bits)      # test_hashattention_top_k.py:160-178


def test_signature_score_closed_form_equals_float_matmul():
    # test_hashattention_top_k.py:225-267: scores == q_sig @ k_sig^T; here also with exact zeros
    g = torch.Generator().manual_seed(2)
    qs = torch.randint(-1, 2, (2, 3, 2, 32), generator=g).float()
    ks = torch.randint(-1, 2, (2, 3, 40, 32), generator=g).float()
    want = torch.matmul(qs, ks.transpose(-2, -1))
    got = O.signature_scores_from_codes(O.pack_signatures(qs), O.pack_signatures(ks))
    assert torch.equal(got.float(), want)
    # no zeros -> bits - 2 * hamming
    qs, ks = qs.sign().where(qs != 0, torch.ones(())), ks.where(ks != 0, torch.ones(()))
    qc, kc = O.pack_signatures(qs), O.pack_signatures(ks)
    ham = torch.zeros(2, 3, 2, 40, dtype=torch.int64)
    x = qc[..., 0].unsqueeze(-1) ^ kc[..., 0].unsqueeze(-2)
    for b in range(32):
        ham += (x >> b) & 1
    assert torch.equal(O.signature_scores_from_codes(qc, kc), 32 - 2 * ham)


def test_hash_topk_cache_growth_and_shrink_error():
    # test_hashattention_top_k.py:180-223, :591-659: only new keys are hashed; a shrinking cache raises
    H, D = 2, 8
    w = _tiny_hat(H, D, 8, 8)
    g = torch.Generator().manual_seed(4)
    q = torch.randn(1, H, 1, D, generator=g)
    k = torch.randn(1, H, 30, D, generator=g)
    m1, sig1 = O.hash_topk(_empty(1, H, 1, 20), q, k[:, :, :20], None, 4, w, "relu")
    m2, sig2 = O.hash_topk(_empty(1, H, 1, 30), q, k, None, 4, w, "relu", key_signatures=sig1)
    _, sig_all = O.hash_topk(_empty(1, H, 1, 30), q, k, None, 4, w, "relu")
    assert sig1.shape[2] == 20 and sig2.shape[2] == 30 and torch.equal(sig2, sig_all)
    assert torch.all((m2.to_dense() != 0).sum(-1) == 4)
    with pytest.raises(ValueError):
        O.hash_topk(_empty(1, H, 1, 20), q, k[:, :, :20], None, 4, w, "relu", key_signatures=sig2)


def test_hash_topk_selected_set_against_brute_force():
    # invariants of test_hashattention_top_k.py:444-589 (exactly k new columns per row, none inside the previous
    # mask, previous columns kept) and the selected SET itself, rebuilt here column by column from the definition:
    # score(j) = sum_e qsig[e] * ksig[j][e], winners = first k of the inactive columns ordered by (-score, j)
    B, Hq, Hkv, Lk, D, k_sel = 2, 4, 2, 37, 8, 5
    w = _tiny_hat(Hq, D, 8, 8, seed=3)
    g = torch.Generator().manual_seed(11)
    q = torch.randn(B, Hq, 1, D, generator=g)
    k = torch.randn(B, Hkv, Lk, D, generator=g)
    add = torch.randn(B, 1, 1, Lk + 3, generator=g).round()  # additive mask, wider than the keys, integer valued
    prev = torch.zeros(B, Hq, 1, Lk)
    prev[..., :3] = 1.0
    prev[..., -4:] = 1.0
    prev[0, 1, 0, 10] = 1.0
    for attention_mask in (None, add):
        m, ksig = O.hash_topk(O.OMask("dense", prev.shape, torch.float32, prev.clone()), q, k, attention_mask, k_sel, w, "silu")
        got = m.to_dense()
        qsig = O.hash_signatures(q, w["query_matrix"], w["query_bias"], "silu")
        for b in range(B):
            for h in range(Hq):
                # key head of query head h is h // G: the signatures of row (b, h) come from K[b, h // 2]
                ks = O.hash_signatures(k[b:b + 1, h // 2:h // 2 + 1].expand(1, 1, Lk, D), [mm[h:h + 1] for mm in w["key_matrix"]],
                                       [bb[h:h + 1] for bb in w["key_bias"]], "silu")[0, 0]
                assert torch.equal(ks, ksig[b, h])
                sc = []
                for j in range(Lk):
                    if prev[b, h, 0, j] != 0:
                        continue
                    val = sum(float(qsig[b, h, 0, e]) * float(ks[j, e]) for e in range(8))
                    if attention_mask is not None:
                        val += float(attention_mask[b, 0, 0, j])
                    sc.append((-val, j))
                winners = {j for _, j in sorted(sc)[:k_sel]}
                active = set(torch.nonzero(got[b, h, 0]).flatten().tolist())
                before = set(torch.nonzero(prev[b, h, 0]).flatten().tolist())
                assert before <= active and active - before == winners and len(winners) == k_sel
                assert torch.all(got[b, h, 0][list(active)] == 1.0)


def test_hash_topk_with_given_signatures_skips_the_mlps():
    # the `key_signatures` / `query_signatures` arguments are what the GPU tests feed the kernels' own codes through
    H, Lk = 2, 12
    ks = torch.ones(1, H, Lk, 4)
    ks[0, 0, 5] = -1.0            # row 0: column 5 is the worst, every other column ties at +4
    ks[0, 1, :, :2] = -1.0        # row 1: all columns tie at 0 except column 7
    ks[0, 1, 7] = 1.0
    qs = torch.ones(1, H, 1, 4)
    m, out = O.hash_topk(_empty(1, H, 1, Lk), torch.zeros(1, H, 1, 3), torch.zeros(1, H, Lk, 3), None, 3, None, "relu",
                         key_signatures=ks, query_signatures=qs)
    assert out is ks
    assert torch.nonzero(m.to_dense()[0, 0, 0]).flatten().tolist() == [0, 1, 2]      # ties: lowest columns first
    assert torch.nonzero(m.to_dense()[0, 1, 0]).flatten().tolist() == [0, 1, 7]      # the best, then the lowest ties


# ------------------------------------------------------------------------- PQCache
def test_pairwise_sq_dist_known_values():
    # utils/test_pq_utils.py:183-209 (and :264-295 batched): all four distances are 1
    x = torch.tensor([[[1.0, 0.0], [0.0, 1.0]]])
    c = torch.tensor([[[0.0, 0.0], [1.0, 1.0]]])
    assert torch.equal(O.pairwise_sq_dist(x, c), torch.ones(1, 2, 2))
    assert O.pairwise_sq_dist(torch.tensor([[[3.0, 4.0]]]), torch.tensor([[[0.0, 0.0]]])).item() == 25.0


def test_kmeans_recovers_two_blobs_and_returns_pre_update_codes():
    # test_pq_utils.py:211-229, :297-322 (well separated blobs) and pq_utils.py:353 vs :399 (code timing)
    g = torch.Generator().manual_seed(0)
    a = torch.randn(1, 50, 2, generator=g) * 0.1 + torch.tensor([5.0, 5.0])
    b = torch.randn(1, 50, 2, generator=g) * 0.1 - torch.tensor([5.0, 5.0])
    X = torch.cat([a, b], dim=1)
    c0 = torch.stack([X[0, 0], X[0, 99]]).unsqueeze(0)
    codes, cent = O.kmeans_lloyd(X, c0, 10)
    assert codes.shape == (1, 100) and codes.dtype == torch.int64 and cent.shape == (1, 2, 2)   # :390-411
    assert torch.all(codes[0, :50] == 0) and torch.all(codes[0, 50:] == 1)
    assert torch.allclose(cent[0, 0], a.mean(1)[0], atol=1e-5) and torch.allclose(cent[0, 1], b.mean(1)[0], atol=1e-5)
    # one iteration: codes are the argmin against the *initial* centres, centres are their means
    c_bad = torch.tensor([[[0.0, 10.0], [0.0, -10.0]]])
    codes1, cent1 = O.kmeans_lloyd(X, c_bad, 1)
    assert torch.equal(codes1, torch.argmin(O.pairwise_sq_dist(X, c_bad), 2))
    assert torch.allclose(cent1[0, 0], X[0][codes1[0] == 0].mean(0), atol=1e-6)


def test_pq_split_against_explicit_loops():
    # pq_top_k.py:216-231: group (b, h, s) holds keys[b, h, init_offset + i, s * d:(s + 1) * d] as its row i
    B, H, Lk, D, n_sub, off = 2, 3, 11, 12, 4, 3
    d = D // n_sub
    keys = torch.arange(B * H * Lk * D, dtype=torch.float32).reshape(B, H, Lk, D)
    X = O.pq_split(keys, off, n_sub)
    assert X.shape == (B * H * n_sub, Lk - off, d)
    for b in range(B):
        for h in range(H):
            for s in range(n_sub):
                grp = (b * H + h) * n_sub + s
                for i in range(Lk - off):
                    assert torch.equal(X[grp, i], keys[b, h, off + i, s * d:(s + 1) * d])


def test_pq_split_ip_against_explicit_loops():
    # pq_top_k.py:219-236 + pq_utils.py:585-612: the same groups, one more coordinate sqrt(phi - |x|^2) with phi the
    # group's largest squared norm; the row that attains phi gets exactly 0
    B, H, Lk, D, n_sub, off = 1, 2, 9, 6, 3, 2
    d = D // n_sub
    g = torch.Generator().manual_seed(5)
    keys = torch.randn(B, H, Lk, D, generator=g)
    X, phi = O.pq_split_ip(keys, off, n_sub)
    assert X.shape == (B * H * n_sub, Lk - off, d + 1) and phi.shape == (B * H * n_sub, 1, 1)
    for h in range(H):
        for s in range(n_sub):
            grp = h * n_sub + s
            sub = [keys[0, h, off + i, s * d:(s + 1) * d] for i in range(Lk - off)]
            norms = [float((v * v).sum()) for v in sub]
            assert math.isclose(float(phi[grp]), max(norms), rel_tol=1e-6)
            for i, v in enumerate(sub):
                assert torch.equal(X[grp, i, :d], v)
                assert math.isclose(float(X[grp, i, d]), math.sqrt(max(max(norms) - norms[i], 0.0)), rel_tol=1e-4, abs_tol=1e-3)
            assert float(X[grp, norms.index(max(norms)), d]) == 0.0
    # keys before init_offset take no part: a huge key there leaves phi alone
    keys2 = keys.clone()
    keys2[:, :, 0] = 100.0
    assert torch.equal(O.pq_split_ip(keys2, off, n_sub)[1], phi)


def test_kmeans_empty_cluster_takes_the_reseed_sample():
    # pq_utils.py:384-396: a cluster without points becomes X[g, random index]; every other centre is the mean of its
    # points. Two groups: in group 0 centre 2 sits far away and stays empty, in group 1 nothing is empty.
    X = torch.tensor([[[0.0, 0.0], [0.0, 2.0], [10.0, 0.0], [10.0, 2.0]],
                      [[0.0, 0.0], [1.0, 0.0], [5.0, 0.0], [9.0, 0.0]]])
    c0 = torch.tensor([[[0.0, 1.0], [9.0, 1.0], [100.0, 100.0]],
                       [[0.0, 0.0], [5.0, 0.0], [9.0, 0.0]]])
    reseed = torch.tensor([[[3, 3, 1], [0, 0, 0]]])      # (iteration, group, centre) -> sample index
    codes, centres = O.kmeans_lloyd(X, c0, iter_limit=1, reseed_idx=reseed)
    assert codes.tolist() == [[0, 0, 1, 1], [0, 0, 1, 2]]
    assert torch.equal(centres[0], torch.tensor([[0.0, 1.0], [10.0, 1.0], [0.0, 2.0]]))   # centre 2 := X[0, 1]
    assert torch.equal(centres[1], torch.tensor([[0.5, 0.0], [5.0, 0.0], [9.0, 0.0]]))    # untouched by the reseed
    with pytest.raises(ValueError):
        O.kmeans_lloyd(X, c0, iter_limit=1)
    # second iteration: the reseeded centre now wins its own sample; codes are those of the assignment BEFORE the
    # last update, centres after it
    reseed2 = torch.cat([reseed, reseed], dim=0)
    codes2, centres2 = O.kmeans_lloyd(X, c0, iter_limit=2, reseed_idx=reseed2)
    assert codes2[0].tolist() == [0, 2, 1, 1]
    assert torch.equal(centres2[0], torch.tensor([[0.0, 0.0], [10.0, 1.0], [0.0, 2.0]]))


def test_ip2l2_augmentation_known_answers():
    # test_pq_utils.py:25-147: phi = largest squared norm of the group, extra column sqrt(phi - ||x||^2),
    # queries get a zero column, and ||x~ - q~||^2 = phi + ||q||^2 - 2 <x, q> (their x = [1,2], q = [3,4])
    g = torch.Generator().manual_seed(8)
    xb = torch.randn(3, 10, 4, generator=g)
    aug, phi = O.ip2l2_augment(xb)
    assert aug.shape == (3, 10, 5) and phi.shape == (3, 1, 1)
    assert torch.equal(aug[..., :4], xb)
    n2 = (xb ** 2).sum(-1)
    assert torch.allclose(phi[:, 0, 0], n2.max(1).values)
    assert torch.allclose(aug[..., 4], (phi[:, :, 0] - n2).sqrt(), atol=1e-6)
    assert torch.allclose((aug ** 2).sum(-1), phi[:, :, 0].expand(3, 10), rtol=1e-5)   # every augmented key has norm^2 phi
    xq = torch.randn(3, 2, 4, generator=g)
    qa = O.ip2l2_augment_queries(xq)
    assert qa.shape == (3, 2, 5) and torch.equal(qa[..., :4], xq) and bool((qa[..., 4] == 0).all())
    x = torch.tensor([[[1.0, 2.0]]])
    q = torch.tensor([[[3.0, 4.0]]])
    xa, ph = O.ip2l2_augment(x)
    l2 = ((xa - O.ip2l2_augment_queries(q)) ** 2).sum().item()
    assert l2 == pytest.approx(ph.item() + 25.0 - 2 * 11.0, rel=1e-5)
    # hence the nearest augmented key is the key of largest inner product
    d = ((aug.unsqueeze(1) - qa.unsqueeze(2)) ** 2).sum(-1)
    assert torch.equal(d.argmin(-1), torch.einsum("gqd,gnd->gqn", xq, xb).argmax(-1))
    # new keys against (d + 1)-wide centroids: zero column appended, plain squared L2, first minimum
    cent = torch.randn(1, 2, 2, 4, 3, generator=g)          # B, Hkv, n_sub, k, d + 1 with d = 2
    nk = torch.randn(1, 2, 3, 4, generator=g)               # B, Hkv, n_new, D = 4
    codes = O.pq_quantize_new(nk, cent)
    assert codes.shape == (1, 3, 2, 2)
    for h in range(2):
        for j in range(3):
            for s_ in range(2):
                v = torch.cat([nk[0, h, j, 2 * s_:2 * s_ + 2], torch.zeros(1)])
                assert int(codes[0, j, h, s_]) == int(((cent[0, h, s_] - v) ** 2).sum(-1).argmin())


def test_pq_scores_manual_and_gqa():
    # test_pq_top_k.py:741-873: score = sum_s q_s . centroid[code]; q head h uses kv head h // G;
    # an augmented last centroid dimension is ignored
    g = torch.Generator().manual_seed(5)
    B, Hq, Hkv, D, n_sub, kc, n = 1, 4, 2, 8, 2, 4, 6
    d = D // n_sub
    q = torch.randn(B, Hq, 1, D, generator=g)
    cent = torch.randn(B, Hkv, n_sub, kc, d + 1, generator=g)
    book = torch.randint(0, kc, (B, n, Hkv, n_sub), generator=g)
    got = O.pq_scores(q, Hkv, cent, book)
    assert got.shape == (B, Hq, 1, n)
    for h in range(Hq):
        for j in range(n):
            want = sum(float(q[0, h, 0, s * d:(s + 1) * d] @ cent[0, h // 2, s, book[0, j, h // 2, s], :d]) for s in range(n_sub))
            assert abs(got[0, h, 0, j].item() - want) < 1e-5


def test_pq_full_attention_rule_and_incremental_codes():
    # test_pq_top_k.py:988-1043 (Lk <= k + offset + Lq + 2^bits) and :515-626 (new keys vs frozen centroids)
    assert O.pq_should_use_full(100, 1, 10, 4, 6) is False      # 100 > 10+4+1+64 = 79
    assert O.pq_should_use_full(79, 1, 10, 4, 6) is True
    g = torch.Generator().manual_seed(6)
    cent = torch.randn(1, 2, 2, 4, 4, generator=g)
    new = torch.randn(1, 2, 3, 8, generator=g)
    codes = O.pq_quantize_new(new, cent)
    assert codes.shape == (1, 3, 2, 2)
    for h in range(2):
        for j in range(3):
            for s in range(2):
                dist = ((new[0, h, j, s * 4:(s + 1) * 4] - cent[0, h, s]) ** 2).sum(-1)
                assert codes[0, j, h, s].item() == int(torch.argmin(dist))


def test_pq_topk_offsets_and_exclusion():
    # test_pq_top_k.py:1208-1306: exactly k new, indices shifted by init_offset, none inside the previous mask
    scores = torch.tensor([[[[0.1, 0.9, 0.8, 0.7, 0.2, 0.6]]]])
    prev = torch.zeros(1, 1, 1, 10)
    prev[..., 3] = 1.0   # column 3 == candidate 1 (offset 2) is already active
    m = O.pq_topk(O.OMask("dense", (1, 1, 1, 10), torch.float32, prev), scores, 2, 2)
    assert torch.nonzero(m.to_dense()[0, 0, 0]).squeeze(-1).tolist() == [3, 4, 5]


# ------------------------------------------------------------- adaptive sampling
def test_adaptive_exp_scores_against_fp64_definition():
    # adaptive_sampling.py:183-197: exp(q.k * scaling + mask - rowmax) over ALL keys, key head h // G, mask cut to Lk
    B, Hq, Hkv, Lk, D = 2, 4, 2, 9, 6
    g = torch.Generator().manual_seed(8)
    q = torch.randn(B, Hq, 1, D, generator=g)
    k = torch.randn(B, Hkv, Lk, D, generator=g)
    add = torch.randn(B, 1, 1, Lk + 2, generator=g)
    scaling = 0.37
    for attention_mask in (None, add):
        got = O.adaptive_exp_scores(q, k, scaling, attention_mask)
        assert got.shape == (B, Hq, 1, Lk) and got.dtype == q.dtype
        for b in range(B):
            for h in range(Hq):
                z = [sum(float(q[b, h, 0, e]) * float(k[b, h // 2, j, e]) for e in range(D)) * scaling for j in range(Lk)]
                if attention_mask is not None:
                    z = [zz + float(attention_mask[b, 0, 0, j]) for j, zz in enumerate(z)]
                top = max(z)
                want = torch.tensor([math.exp(zz - top) for zz in z], dtype=torch.float64)
                assert torch.allclose(got[b, h, 0].double(), want, rtol=1e-5, atol=1e-7)
                assert float(got[b, h, 0].max()) == 1.0
    # the result is in the query dtype (the reference never widens here)
    assert O.adaptive_exp_scores(q.bfloat16(), k.bfloat16(), scaling, None).dtype == torch.bfloat16


def test_adaptive_range_and_base_count():
    # sampling/implementations/test_adaptive_sampling.py:207-272
    assert O.adaptive_sampling_range(131072, 128, 1024) == (128, 130048, 129920)
    assert O.adaptive_sampling_range(100, 0.1, 0.2) == (10, 80, 70)
    assert O.adaptive_base_count(0.01, 129920) == 1299
    assert O.adaptive_base_count(0.001, 100) == 2 and O.adaptive_base_count(5, 100) == 5


def test_adaptive_budget_closed_form():
    # adaptive_sampling.py:282-302 with hand-picked numbers
    expw = torch.tensor([[[[0.0, 1.0, 3.0, 1.0, 3.0, 0.0]]]])
    base = torch.tensor([[[[1, 2, 3, 4]]]])           # draws 1,3,1,3 -> unbiased std = sqrt(4/3)
    budget, p = O.adaptive_budget(_empty(1, 1, 1, 6), expw, base, 1, 5, 0.5, 0.5)
    # delta = 0.5 -> ppf(0.5) = 0 -> budget_squared = 0 -> clamp to 1 -> clamp to n_base = 4
    assert budget.item() == 4 and abs(p.item() - 1.0) < 1e-6
    budget, _ = O.adaptive_budget(_empty(1, 1, 1, 6), expw, base, 1, 5, 0.05, 0.05)
    assert budget.item() == 4                          # clamp to the range size


# ----------------------------------------------------------------------- attention
def test_sink_logit_closed_form():
    # utils/test_mask_attention_utils.py:1025-1140: [1/2,1/2] -> [1/3,1/3], weights sum 2/3
    q = torch.zeros(1, 1, 2, 2)
    k = torch.zeros(1, 1, 2, 2)
    v = torch.tensor([[[[1.0, 0.0], [0.0, 1.0]]]])
    full = O.OMask.full((1, 1, 2, 2), torch.float32)
    out, w = O.masked_attention(q, k, v, None, None, 1.0, full)
    assert out.shape == (1, 2, 1, 2) and torch.allclose(out, torch.full((1, 2, 1, 2), 0.5))
    out, w = O.masked_attention(q, k, v, None, torch.tensor([0.0]), 1.0, full)
    assert torch.allclose(out, torch.full((1, 2, 1, 2), 1.0 / 3.0), atol=1e-6)
    assert torch.allclose(w.sum(-1), torch.full((1, 1, 2), 2.0 / 3.0), atol=1e-6)


def test_empty_mask_equals_hf_eager_attention():
    # test_mask_attention_utils.py:718-955: empty mask == transformers eager_attention_forward (GQA, Lq != Lk)
    from transformers.models.llama.modeling_llama import eager_attention_forward

    g = torch.Generator().manual_seed(7)
    B, Hq, Hkv, Lq, Lk, D = 2, 4, 2, 3, 9, 8
    q = torch.randn(B, Hq, Lq, D, generator=g)
    k = torch.randn(B, Hkv, Lk, D, generator=g)
    v = torch.randn(B, Hkv, Lk, D, generator=g)
    am = torch.zeros(B, 1, Lq, Lk)
    am[..., -2:] = torch.finfo(torch.float32).min

    class M(torch.nn.Module):
        num_key_value_groups = Hq // Hkv

    mod = M().eval()
    want, want_w = eager_attention_forward(mod, q, k, v, am, scaling=D ** -0.5, dropout=0.0)
    got, got_w = O.masked_attention(q, k, v, am, None, D ** -0.5, O.OMask.empty((B, Hq, Lq, Lk), torch.float32))
    assert torch.allclose(got, want, atol=1e-6) and torch.allclose(got_w, want_w, atol=1e-6)


def test_weighted_mask_exp_weights_formula():
    # test_mask_attention_utils.py:454-562: kept entries are exp(logit - rowmax) / weight, others 0
    g = torch.Generator().manual_seed(8)
    q = torch.randn(1, 2, 4, 8, generator=g)
    k = torch.randn(1, 2, 6, 8, generator=g)
    v = torch.randn(1, 2, 6, 8, generator=g)
    dm = torch.randint(0, 3, (1, 2, 4, 6), generator=g).float()
    dm[..., 0] = 1.0
    out, w = O.masked_attention(q, k, v, None, None, 0.3, O.OMask("dense", (1, 2, 4, 6), torch.float32, dm))
    logits = torch.matmul(q, k.transpose(-2, -1)) * 0.3
    e = torch.exp(logits - logits.max(-1, keepdim=True)[0])
    e = torch.where(dm != 0, e / (dm + 1e-6), torch.zeros(()))
    want = torch.matmul(e / e.sum(-1, keepdim=True), v).transpose(1, 2)
    assert torch.allclose(out, want, atol=1e-6)
    assert torch.all(w[dm == 0] == 0)


def test_chain_composition_on_brute_forceable_size():
    # no reference test covers maskers -> output; composed from the pinned pieces and checked by brute force
    g = torch.Generator().manual_seed(9)
    B, Hq, Hkv, Lk, D = 2, 4, 2, 64, 16
    q = torch.randn(B, Hq, 1, D, generator=g)
    k = torch.randn(B, Hkv, Lk, D, generator=g)
    v = torch.randn(B, Hkv, Lk, D, generator=g)
    out, w, m = O.research_attention([("sink", 4), ("local", 8), ("oracle_topk", 6)], q, k, v, None, D ** -0.5)
    for b in range(B):
        for h in range(Hq):
            kk, vv = k[b, h // 2].double(), v[b, h // 2].double()
            s = (kk @ q[b, h, 0].double())
            fixed = set(range(4)) | set(range(Lk - 8, Lk))
            rest = sorted((j for j in range(Lk) if j not in fixed), key=lambda j: (-float(q[b, h, 0] @ k[b, h // 2, j]), j))[:6]
            sel = sorted(fixed | set(rest))
            p = torch.softmax(s[sel] * D ** -0.5, 0)
            want = (p.unsqueeze(1) * vv[sel]).sum(0)
            assert torch.allclose(out[b, 0, h].double(), want, atol=1e-5)
            assert torch.nonzero(m.to_dense()[b, h, 0]).squeeze(-1).tolist() == sel


def test_usa_checkpoint_conversion_matches_the_linear_modules(tmp_path):
    """A USA-style state dict of per-head nn.Sequential MLPs converts to matrices that reproduce the modules'
    outputs (y = x W^T + b -> x @ matrix + bias) and survives the HAT file round trip (hashattention_utils.py:9-180)."""
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import (
        convert_usa_weights_to_hash_attention, create_hat_weights_file_from_usa, load_hat_weights)

    torch.manual_seed(0)
    layers, heads, d, hidden, bits = 2, 3, 8, 16, 4
    state, modules = {}, {}
    for layer in range(layers):
        for tag in ("q", "k"):
            for head in range(heads):
                seq = torch.nn.Sequential(torch.nn.Linear(d, hidden), torch.nn.SiLU(), torch.nn.Linear(hidden, hidden),
                                          torch.nn.SiLU(), torch.nn.Linear(hidden, bits, bias=(tag == "q")))
                modules[(layer, tag, head)] = seq
                for name, value in seq.state_dict().items():
                    state[f"{layer}.learning_to_hash_transformation_{tag}.{head}.{name}"] = value
    hat = convert_usa_weights_to_hash_attention(state, num_layers=layers, num_heads=heads, num_mlp_layers=3)
    assert sorted(hat) == [0, 1]
    assert [tuple(m.shape) for m in hat[0]["key_matrix"]] == [(heads, d, hidden), (heads, hidden, hidden), (heads, hidden, bits)]
    assert torch.all(hat[1]["key_bias"][2] == 0)           # the key MLPs' last layer has no bias: zeros
    x = torch.randn(1, heads, 5, d)
    for layer in range(layers):
        for tag, kind in (("q", "query"), ("k", "key")):
            sig = O.hash_signatures(x, hat[layer][f"{kind}_matrix"], hat[layer][f"{kind}_bias"], "silu")
            for head in range(heads):
                want = torch.sign(modules[(layer, tag, head)](x[0, head]))
                assert torch.equal(sig[0, head], want)
    path = tmp_path / "hat.pkl"
    create_hat_weights_file_from_usa(state, str(path), num_layers=layers, num_heads=heads)
    again = load_hat_weights(str(path))
    for layer in range(layers):
        for name in ("query_matrix", "query_bias", "key_matrix", "key_bias"):
            for a, b in zip(hat[layer][name], again[layer][name]):
                assert torch.equal(a, b)


def test_hat_weight_loader_runs_no_code_from_the_file(tmp_path):
    # file format of the reference (utils/hashattention_utils.py:155-180): a pickle of Dict[layer] -> Dict[name] ->
    # List[Tensor]. The loader resolves tensors and plain containers only.
    import pickle

    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import (
        load_hat_weights, random_hat_weights, save_hat_weights)

    w = random_hat_weights(2, 3, 8, 4, 2, 6, dtype=torch.bfloat16, seed=3)
    w[1]["key_bias"][0] = torch.nn.Parameter(w[1]["key_bias"][0].float(), requires_grad=False)  # trained files hold these
    good = tmp_path / "hat.pkl"
    with open(good, "wb") as f:                      # written as the reference writes it: a bare pickle.dump
        pickle.dump(w, f)
    back = load_hat_weights(str(good))
    assert sorted(back) == [0, 1]
    for layer in w:
        for name in w[layer]:
            assert len(back[layer][name]) == len(w[layer][name])
            for a, b in zip(back[layer][name], w[layer][name]):
                assert a.dtype == b.dtype and torch.equal(a, b.detach())
    save_hat_weights(w, str(tmp_path / "again.pkl"))
    assert torch.equal(load_hat_weights(str(tmp_path / "again.pkl"))[0]["query_matrix"][1], w[0]["query_matrix"][1])

    marker = tmp_path / "ran"

    class Payload:
        def __reduce__(self):
            return (open, (str(marker), "w"))

    bad = tmp_path / "bad.pkl"
    with open(bad, "wb") as f:
        pickle.dump({0: {"query_matrix": [Payload()]}}, f)
    with pytest.raises(pickle.UnpicklingError, match="only plain containers of tensors"):
        load_hat_weights(str(bad))
    assert not marker.exists()
    with open(bad, "wb") as f:
        pickle.dump([1, 2, 3], f)
    with pytest.raises(ValueError, match="expected Dict"):
        load_hat_weights(str(bad))


def test_dropout_keep_follows_the_counter_layout_and_the_rate():
    """The fate of entry (row r, column j): word 0 of Philox4x32-10 with counter (j, r, offset lo, offset hi) and key
    (seed lo, seed hi), kept when it is at least p * 2^32. Checked against single calls of the Philox function (which the
    Random123 vectors pin), so a swapped row / column or a wrong word fails; and the kept share is 1 - p."""
    import numpy as np

    seed, offset, p = 0x1234_5678_9ABC_DEF0, (5 << 32) | 77, 0.3
    keep = O.dropout_keep(seed, offset, 6, 40, p)
    key = (seed & 0xFFFFFFFF, seed >> 32)
    for r, j in ((0, 0), (1, 0), (0, 1), (5, 39), (3, 17)):
        u = O.philox4x32_10(np.array([[j, r, offset & 0xFFFFFFFF, offset >> 32]], dtype=np.uint64), key)[0, 0]
        assert bool(keep[r, j]) == (int(u) >= int(p * 2 ** 32)), (r, j)
    big = O.dropout_keep(seed, offset, 64, 4096, p)
    assert abs(float(big.float().mean()) - (1 - p)) < 0.005
    assert not torch.equal(O.dropout_keep(seed, offset + 1, 6, 40, p), keep)      # another call, another stream
    assert not torch.equal(O.dropout_keep(seed + 1, offset, 6, 40, p), keep)


def test_masked_attention_dropout_has_the_form_of_torch_dropout():
    """torch.nn.functional.dropout zeroes an element with probability p and scales the others by 1 / (1 - p)
    (mask_attention_utils.py:234-238 applies it to the exp weights, before numerator and denominator). The oracle's
    probabilities with dropout, times their denominator, are therefore 0 or the undropped exp weight / (1 - p); the output
    is the softmax over the kept entries; the sink term is not scaled."""
    g = torch.Generator().manual_seed(3)
    B, H, Lq, Lk, D, p = 1, 2, 2, 50, 8, 0.4
    q, k, v = (torch.randn(B, H, n, D, generator=g) for n in (Lq, Lk, Lk))
    dense = torch.zeros(B, H, Lq, Lk)
    dense[..., ::3] = 1.0
    dense[..., 1] = 0.5
    m = O.OMask("dense", tuple(dense.shape), dense.dtype, dense)
    sinks = torch.tensor([0.3, -0.2])
    drop = (p, 11, 5)
    out0, w0 = O.masked_attention(q, k, v, None, sinks, 0.5, m)
    out1, w1 = O.masked_attention(q, k, v, None, sinks, 0.5, m, dropout=drop)
    keep = O.dropout_keep(11, 5, B * H * Lq, Lk, p).view(B, H, Lq, Lk)
    assert torch.equal(w1 != 0, (w0 != 0) & keep)
    # by hand, in fp64: e = exp(z - max) / (w + 1e-6) on the mask, times keep / (1 - p); den += exp(sink - max)
    z = torch.matmul(q.double(), k.double().transpose(2, 3)) * 0.5
    mx = z.max(dim=-1, keepdim=True)[0]
    e = torch.exp(z - mx) * torch.where(dense != 0, 1.0 / (dense.double() + 1e-6), torch.zeros(()).double())
    e = e * keep.double() / (1.0 - float(torch.tensor(p, dtype=torch.float32)))
    srow = sinks.double().view(1, H, 1, 1)
    nm = torch.maximum(mx, srow)
    sc = torch.exp(mx - nm)
    den = e.sum(-1, keepdim=True) * sc + torch.exp(srow - nm)
    want = (torch.matmul(e, v.double()) * sc / den).transpose(1, 2)
    assert torch.allclose(out1.double(), want, rtol=1e-5, atol=1e-6)
    assert not torch.allclose(out1, out0, rtol=1e-3)


def test_masked_attention_dropout_of_the_normalised_probabilities():
    """The reference's dense path is scaled_dot_product_attention(dropout_p=...) (mask_attention_utils.py:40-52):
    softmax first, then dropout of the probabilities, then the product with V. `dropout_numerator_only` must be exactly
    that: torch.softmax in fp64, the oracle's own keep mask scaled by 1 / (1 - p), times V - and differ from the form that
    drops before the denominator."""
    g = torch.Generator().manual_seed(4)
    B, H, Lq, Lk, D, p = 1, 2, 2, 40, 8, 0.3
    q, k, v = (torch.randn(B, H, n, D, generator=g) for n in (Lq, Lk, Lk))
    empty = O.OMask.empty((B, H, Lq, Lk), torch.float32)
    drop = (p, 21, 9)
    out, w = O.masked_attention(q, k, v, None, None, 0.5, empty, dropout=drop, dropout_numerator_only=True)
    keep = O.dropout_keep(21, 9, B * H * Lq, Lk, p).view(B, H, Lq, Lk)
    probs = torch.softmax(torch.matmul(q.double(), k.double().transpose(2, 3)) * 0.5, dim=-1)
    dropped = probs * keep.double() / (1.0 - float(torch.tensor(p, dtype=torch.float32)))
    want = torch.matmul(dropped, v.double()).transpose(1, 2)
    assert torch.allclose(out.double(), want, rtol=1e-5, atol=1e-6)
    assert torch.allclose(w.double(), dropped, rtol=1e-5, atol=1e-7)
    other, _ = O.masked_attention(q, k, v, None, None, 0.5, empty, dropout=drop)
    assert not torch.allclose(out, other, rtol=1e-3)
