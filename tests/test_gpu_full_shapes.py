"""GPU parity at the sizes the benchmark runs: the code paths that only large shapes reach (the one-kernel
HashAttention decode step at 256 rows x 32768 keys, the Lloyd assignment on the matrix cores with 256 centres,
the stand-alone lookup-table kernel of the PQ scoring beyond 65536 candidates, the QK scoring pass and the 16-bit
selection at 131072 keys), each against the CPU oracle on the same seeded inputs, through the C ABI."""
import pytest
import torch

from _util import make_qkv, rel_err
from oracle import reference_path as O

pytestmark = pytest.mark.gpu


def _sa():
    import sparse_attention_hub_amd.sparse_attention as sa

    return sa


def _unpack_codes(codes, bits=32):
    """{-1, 0, +1} signatures (float32, CPU) from two-plane codes (..., 2) int32."""
    c = codes.cpu().to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(bits)
    pos = (c[..., 0].unsqueeze(-1) >> shifts) & 1
    nonzero = (c[..., 1].unsqueeze(-1) >> shifts) & 1
    return ((pos * 2 - 1) * nonzero).float()


def test_config3_step_is_one_kernel_and_matches_the_oracle(cuda):
    """headline configuration 3 at its full shape (batch 8, 32 query / 8 KV heads, 32768 keys, bf16, Sink 128 + Local 512 +
    HashAttention top-2048): the warm decode step is ONE launch of k_hash_decode_attn, every row holds
    128 + 512 + 2048 distinct columns, and for batch rows 0 and 7 the selected sets are bit-identical to the
    oracle's (scoring the kernel's own signatures) and the outputs agree within the bf16 bar."""
    from sparse_attention_hub_amd import _native as N
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    sa = _sa()
    B, Hq, Hkv, Lk, D = 8, 32, 8, 32768, 128
    sink, window, heavy = 128, 512, 2048
    dtype = torch.bfloat16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=31)
    q0 = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=32)[0]
    wts = random_hat_weights(1, Hq, D, 32, 3, 128, dtype=dtype, seed=1)
    cfg = sa.HashAttentionTopKMaskerConfig(heavy_size=heavy, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                           hat_mlp_activation="silu", hat_weights=wts)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=sink), sa.LocalMaskerConfig(window_size=window), cfg]))
    ra.return_attention_weights = False
    meta = {}
    kc, vc = k.to(cuda), v.to(cuda)
    scaling = D ** -0.5
    # cold call on all but the last two keys: hashes them (general path); a first decode step brings the compact
    # code stream up to date (one more launch, once); then the warm step on all keys
    for n in (Lk - 2, Lk - 1):
        ra.custom_attention(None, q0.to(cuda), kc[:, :, :n], vc[:, :, :n], None, scaling, 0.0, sparse_meta_data=meta, layer_idx=0)
    torch.cuda.synchronize()
    N.timing_enable(True)
    out, _ = ra.custom_attention(None, q.to(cuda), kc, vc, None, scaling, 0.0, sparse_meta_data=meta, layer_idx=0)
    torch.cuda.synchronize()
    launches = N.timing_collect()
    N.timing_enable(False)
    assert set(launches) == {"k_hash_decode_attn"} and launches["k_hash_decode_attn"][0] == 1, launches
    plan = next(iter(ra._plans.values()))
    total = sink + window + heavy
    assert bool((plan.cnt.cpu() == total).all())
    cols = plan.cols[:, :total].long()
    srt = torch.sort(cols, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all()) and int(cols.min()) == 0 and int(cols.max()) == Lk - 1
    cache = meta["key"][0]
    assert cache.n == Lk - 2          # the newest keys sit inside the local window: hashed with the next block of 64
    # the query signatures, from the stand-alone signature kernel (same order of sums, same bits as inside the step)
    qcodes = torch.empty((B * Hq, 2), dtype=torch.int32, device=cuda)
    ra.maskers[2]._hash(q.to(cuda), Hq, Hq, 0, 1, 0, "query", qcodes, 1, 0)
    qsig = _unpack_codes(qcodes).view(B, Hq, 1, 32)
    specs = [("sink", sink), ("local", window), ("hash_topk", heavy, wts[0], "silu")]
    member = torch.zeros((B * Hq, Lk), dtype=torch.bool, device=cuda)
    member.scatter_(1, cols, True)
    member = member.cpu().view(B, Hq, Lk)
    for b in (0, B - 1):
        ksig = _unpack_codes(cache.codes[b:b + 1, :, :cache.n])
        state = {"key_sig": ksig, "query_sig": qsig[b:b + 1]}
        oo, _, om = O.research_attention(specs, q[b:b + 1], k[b:b + 1], v[b:b + 1], None, scaling, state=state)
        assert torch.equal(member[b], om.to_dense()[0, :, 0] != 0), f"batch row {b}: selected sets differ"
        err = rel_err(out[b], oo[0])
        assert err < 2e-2, f"batch row {b}: output rel err {err}"


def test_lloyd_steps_with_256_centres_match_the_oracle(cuda):
    """The matrix-core assignment kernel in the benchmark's geometry (sub-vectors of 8, 256 centres, 8 centre
    tiles) against the oracle's Lloyd step, one (batch, KV head) slice = 16 groups of 4096 keys. Each of three
    steps starts from the ORACLE's centres, so a disagreement cannot compound: codes agree except at near-ties
    (the kernel expands |x - c|^2 into |x|^2 - 2 x.c + |c|^2, the reference sums squared differences), and every
    centre whose members agree matches to fp32 accumulation tolerance."""
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.utils.pq_utils import (
        gather_sub_vectors, kmeans_keys_batched, seeded_initial_centres,
    )

    B, Hkv, n, D, n_sub, n_cent = 1, 1, 4096, 128, 16, 256
    d_sub = D // n_sub
    k = make_qkv(B, Hkv, Hkv, 1, n, D, torch.bfloat16, outliers=True, seed=41)[1]
    X = O.pq_split(k, 0, n_sub)                                       # (16, 4096, 8)
    start = seeded_initial_centres(n_sub, n, n_cent, 5, torch.device("cpu"))
    centres = gather_sub_vectors(k, 0, n_sub, start)                  # (16, 256, 8) fp32
    reseed = torch.randint(0, n, (1, n_sub, n_cent), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    kc = k.to(cuda)
    for it in range(3):
        codes_o, new_o = O.kmeans_lloyd(X.float(), centres, 1, reseed_idx=reseed)
        codes = torch.zeros((B, Hkv, n, n_sub), dtype=torch.uint8, device=cuda)
        new_k, _ = kmeans_keys_batched(kc, 0, n_sub, n_cent, 1, codes, n, cluster_centers=centres.to(cuda), seed=0)
        got = codes[0, 0].cpu().long().t()                             # (16, 4096)
        same = got == codes_o
        assert same.float().mean().item() >= 0.995, same.float().mean().item()
        # where they differ, the two centres are (nearly) equally far from the key
        g_i, n_i = torch.nonzero(~same, as_tuple=True)
        if g_i.numel():
            x = X.float()[g_i, n_i]
            da = ((x - centres[g_i, got[g_i, n_i]]) ** 2).sum(-1)
            db = ((x - centres[g_i, codes_o[g_i, n_i]]) ** 2).sum(-1)
            assert bool(((da - db).abs() <= 1e-3 * torch.maximum(da, db) + 1e-5).all())
        # centres of clusters with identical membership
        agree = torch.ones(n_sub, n_cent, dtype=torch.bool)
        for g in range(n_sub):
            bad = torch.cat([got[g][~same[g]], codes_o[g][~same[g]]])
            agree[g, bad] = False
        assert agree.float().mean().item() > 0.9
        assert torch.allclose(new_k.cpu()[agree], new_o.float()[agree], rtol=1e-4, atol=1e-4)
        centres = new_o.float()


def test_reference_named_kmeans_and_reconstruction_error_bars(cuda):
    """`kmeans_batched_pytorch` / `kmeans_batched` / `compute_reconstruction_errors` under the reference's names,
    and its quality bars (tests/unit/.../implementations/test_pq_top_k.py:173-196, :359-513): relative
    reconstruction error below 1, falling as the number of centres grows from 2 to 128."""
    sa = _sa()
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.utils.pq_utils import (
        compute_reconstruction_errors, kmeans_batched, kmeans_batched_pytorch,
    )

    g = torch.Generator().manual_seed(42)
    keys = torch.randn(1, 1, 128, 16, generator=g)
    errs = {}
    for metric in ("euclidean", "ip"):
        for bits in (1, 2, 3, 4, 5, 6, 7):
            masker = sa.PQCache(sa.PQCacheConfig(heavy_size=10, pq_group_factor=8, pq_bits=bits, kmeans_iter=100,
                                                 init_offset=0, metric=metric))
            meta = {}
            masker._initialize_pq_cache(meta, 0)
            cent, book = masker._perform_kmeans_clustering(keys.to(cuda), 0, meta)
            e = compute_reconstruction_errors(keys.to(cuda), cent, book, 2, use_ip_metric=metric == "ip")
            assert set(e) == {"mse_error", "l2_error", "relative_error"} and e["relative_error"] < 1.0
            errs[(metric, bits)] = e["relative_error"]
        assert errs[(metric, 1)] > errs[(metric, 4)] > errs[(metric, 7)]
    assert errs[("euclidean", 7)] < 1e-6          # 128 centres for 128 keys: every key is its own centre
    # the generic entry points: two well-separated blobs per group are recovered, shapes and dtypes as the
    # reference returns them (tests/unit/sparse_attention/utils/test_pq_utils.py:211-229, :297-322, :390-411)
    blobs = torch.cat([torch.randn(3, 50, 4, generator=g) * 0.1 + 5.0, torch.randn(3, 50, 4, generator=g) * 0.1 - 5.0], dim=1)
    cent, codes = kmeans_batched_pytorch(blobs.to(cuda), 2, 10)
    assert cent.shape == (3, 2, 4) and codes.shape == (3, 100) and codes.dtype == torch.int64 and cent.dtype == torch.float32
    for gi in range(3):
        c = codes[gi].cpu()
        assert len(set(c[:50].tolist())) == 1 and len(set(c[50:].tolist())) == 1 and c[0] != c[99]
        near = cent[gi].cpu().abs().mean(-1)
        assert torch.allclose(near, torch.full((2,), 5.0), atol=0.2)
    given = torch.tensor([[[5.0] * 4, [-5.0] * 4]] * 3)
    choice, centres = kmeans_batched(blobs.to(cuda), 2, cluster_centers=given.to(cuda), iter_limit=5)
    assert bool((choice[:, :50] == 0).all()) and bool((choice[:, 50:] == 1).all())
    want = torch.stack([blobs[:, :50].mean(1), blobs[:, 50:].mean(1)], dim=1)
    assert torch.allclose(centres.cpu(), want, atol=1e-4)
    with pytest.raises(ValueError, match="Expected 3D input"):
        kmeans_batched(blobs[0].to(cuda), 2)
    with pytest.raises(NotImplementedError):
        kmeans_batched(blobs.to(cuda), 2, distance="cosine")
    with pytest.raises(ValueError, match="cluster_centers shape mismatch"):
        kmeans_batched(blobs.to(cuda), 2, cluster_centers=given[:, :1].to(cuda))


def test_pq_chain_beyond_65536_candidates_builds_the_table_in_its_own_launch(cuda):
    """More than 65536 candidate keys: the lookup table no longer fits the scoring workgroups' own build and comes
    from k_pq_lut. Scores, selection and attention against the oracle given the kernel's codebook."""
    from sparse_attention_hub_amd import _native as N

    sa = _sa()
    B, Hq, Hkv, Lk, D = 1, 8, 2, 70000, 128
    off, window, heavy, n_sub, bits = 16, 64, 300, 16, 8
    dtype = torch.bfloat16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, outliers=True, seed=51)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[
        sa.SinkMaskerConfig(sink_size=off), sa.LocalMaskerConfig(window_size=window),
        sa.PQCacheConfig(heavy_size=heavy, pq_group_factor=n_sub, pq_bits=bits, kmeans_iter=2, init_offset=off, metric="euclidean")]))
    meta = {}
    N.timing_enable(True)
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    torch.cuda.synchronize()
    launches = N.timing_collect()
    N.timing_enable(False)
    assert "k_pq_lut" in launches and "k_pq_adc" in launches, launches
    cent = meta["pq_centroids"][0].cpu()
    codes = meta["pq_codebook"][0].to_reference().cpu()
    assert codes.shape == (B, Lk - off, Hkv, n_sub)
    oo, ow, om = O.research_attention([("sink", off), ("local", window), ("pq_topk", heavy, off, cent, codes)], q, k, v, None, D ** -0.5)
    assert torch.equal(w.cpu() != 0, om.to_dense() != 0)
    assert rel_err(out, oo) < 2e-2
    # a warm step through the decode plan at the same size
    ra.return_attention_weights = False
    q2, kn, vn = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=52)
    k2, v2 = torch.cat([k, kn], 2), torch.cat([v, vn], 2)
    N.timing_enable(True)
    out2, _ = ra.custom_attention(None, q2.to(cuda), k2.to(cuda), v2.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    torch.cuda.synchronize()
    launches = N.timing_collect()
    N.timing_enable(False)
    assert "k_pq_lut" in launches, launches
    # the plan quantises new keys a block at a time: the key appended by this step lies inside the local window
    # and is still pending; the oracle scores it with the code the general path would give it (its column is
    # active, so the score never matters)
    assert meta["pq_codebook"][0].n == Lk - off
    codes2 = torch.cat([codes, O.pq_quantize_new(kn, cent)], dim=1)
    oo2, _, _ = O.research_attention([("sink", off), ("local", window), ("pq_topk", heavy, off, cent, codes2)], q2, k2, v2, None, D ** -0.5)
    assert rel_err(out2, oo2) < 2e-2
    # the general path (attention weights requested) catches up on the pending key
    ra.return_attention_weights = True
    ra.custom_attention(None, q2.to(cuda), k2.to(cuda), v2.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    assert torch.equal(meta["pq_codebook"][0].to_reference().cpu(), codes2)


def test_oracle_topk_at_131072_keys_matches_matmul_and_stable_sort(cuda):
    """Config 5's context length on one KV group (4 query heads): the QK scoring pass and the 16-bit selection at
    131072 keys against `torch.matmul` in bf16 and a stable descending sort on the CPU, then the attention over
    the selected rows."""
    sa = _sa()
    B, Hq, Hkv, Lk, D = 1, 4, 1, 131072, 128
    sink, window = 128, 1024
    heavy = int(0.02 * Lk)
    dtype = torch.bfloat16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, outliers=True, seed=61)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[
        sa.SinkMaskerConfig(sink_size=sink), sa.LocalMaskerConfig(window_size=window), sa.OracleTopKConfig(heavy_size=0.02)]))
    ra.return_attention_weights = False
    out, _ = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data={}, layer_idx=0)
    torch.cuda.synchronize()
    plan = next(iter(ra._plans.values()))
    total = sink + window + heavy
    assert bool((plan.cnt.cpu() == total).all())
    member = torch.zeros((Hq, Lk), dtype=torch.bool, device=cuda)
    member.scatter_(1, plan.cols[:, :total].long(), True)
    oo, _, om = O.research_attention([("sink", sink), ("local", window), ("oracle_topk", 0.02)], q, k, v, None, D ** -0.5)
    want = om.to_dense()[0, :, 0] != 0
    got = member.cpu()
    # the scores themselves: bf16 rounding of an fp32 accumulation; torch's CPU matmul may round a value that sits
    # on a rounding boundary the other way, which can swap two neighbours at the threshold: at least 99.9 % overlap
    overlap = (got & want).sum().item() / want.sum().item()
    assert overlap >= 0.999, overlap
    assert bool(got[:, :sink].all()) and bool(got[:, Lk - window:].all())
    assert rel_err(out, oo) < 2e-2


@pytest.mark.parametrize("Lk,window", [(131072, 1024)])
def test_adaptive_chain_at_131072_keys_keeps_the_denominator_guarantee(cuda, Lk, window):
    """Config 5's chain (Sink + Local + OracleTopK 2 % + AdaptiveSampling 1 %) at 131072 keys, one batch row:
    the importance-weighted sum over the final mask estimates the full softmax denominator within epsilon for at
    least (1 - delta) of the rows (with slack for the normal approximation); entries distinct and in range."""
    sa = _sa()
    B, Hq, Hkv, Lq, D = 1, 32, 8, 1, 128
    eps, delta = 0.1, 0.1
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, torch.bfloat16, seed=23, outliers=False, device=cuda)
    q = q * 0.5
    cfgs = [sa.SinkMaskerConfig(sink_size=128), sa.LocalMaskerConfig(window_size=window), sa.OracleTopKConfig(heavy_size=0.02),
            sa.AdaptiveSamplingMaskerConfig(base_rate_sampling=0.01, epsilon=eps, delta=delta, init_offset=128, local_offset=window)]
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    mask = sa.Mask.create_empty_mask((B, Hq, Lq, Lk), torch.bfloat16, cuda)
    scaling = D ** -0.5
    scratch = {}
    for m in ra.maskers:
        mask = m.add_mask(k, q, v, None, scaling, 0.0, {}, mask, layer_idx=0, _call_scratch=scratch)
    rows = mask.rows
    torch.cuda.synchronize()
    cnt = rows.cnt.long().cpu()
    budget = ra.maskers[-1].last_budget.long().cpu()
    n = Lk - 128 - window
    fixed = 128 + window + int(0.02 * Lk)
    assert int(budget.min()) >= int(0.01 * n) and int(budget.max()) <= n
    assert bool((cnt <= fixed + budget).all()) and bool((cnt > fixed).all())
    kk = k.double().repeat_interleave(Hq // Hkv, dim=1)
    z = torch.matmul(q.double(), kk.transpose(-1, -2)) * scaling
    e = torch.exp(z - z.amax(dim=-1, keepdim=True)).reshape(B * Hq, Lk)
    true_den = e.sum(dim=-1)
    cols = rows.cols.long()
    pos = torch.arange(rows.cap, device=cuda).unsqueeze(0)
    valid = pos < rows.cnt.long().unsqueeze(1)
    wts = rows.w.double()
    est = torch.where(valid, torch.gather(e, 1, cols.clamp(0, Lk - 1)) / wts.clamp_min(1e-9), torch.zeros_like(wts)).sum(dim=-1)
    rel = ((est - true_den).abs() / true_den).cpu()
    assert float((rel <= eps).double().mean()) >= 1.0 - delta - 0.1, float((rel <= eps).double().mean())
    big = torch.where(valid, cols, torch.full_like(cols, Lk + 1) + pos)
    srt = torch.sort(big, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all())
    assert bool(((cols >= 0) & (cols < Lk) | ~valid).all())
    # and the attention over that weighted mask against the oracle given the same mask
    from sparse_attention_hub_amd.sparse_attention.utils.mask_attention_utils import get_masked_attention_output

    out = get_masked_attention_output(None, q, k, v, None, None, scaling, 0.0, mask)
    dense = mask.get_dense_mask().cpu()
    oo, _ = O.masked_attention(q.cpu(), k.cpu(), v.cpu(), None, None, scaling,
                               O.OMask("dense", tuple(dense.shape), torch.bfloat16, dense))
    assert rel_err(out, oo) < 2e-2


@pytest.mark.parametrize("d,k", [(24, 64), (64, 64), (100, 16), (128, 256)])
def test_kmeans_batched_on_wide_vectors_matches_the_oracle(cuda, d, k):
    """`kmeans_batched` (pq_utils.py:260-438) on vectors wider than the 16 dimensions of the headline geometry: the
    matrix-core assignment pads the contraction to the next of 32 / 64 / 128 dimensions, and 256 centres of 128
    dimensions take their sums in a launch of their own. Three Lloyd steps from shared start centres against the
    oracle; keys whose two nearest centres are (nearly) equally far may take the other one."""
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.utils.pq_utils import (
        kmeans_batched,
    )

    b, n = 3, 3000
    g = torch.Generator().manual_seed(60 + d)
    X = torch.randn(b, n, d, generator=g) + 2.0 * torch.randn(b, 1, d, generator=g)
    start = torch.stack([X[i, torch.randperm(n, generator=g)[:k]] for i in range(b)])
    centres_in = start
    for _ in range(3):                      # every step starts from the ORACLE's centres, so a disagreement cannot compound
        codes_o, cent_o = O.kmeans_lloyd(X, centres_in, 1)
        choice, centres = kmeans_batched(X.to(cuda), k, cluster_centers=centres_in.to(cuda), iter_limit=1)
        assert choice.shape == (b, n) and choice.dtype == torch.int64 and centres.shape == (b, k, d)
        got = choice.cpu()
        same = got == codes_o
        assert same.float().mean().item() >= 0.995, same.float().mean().item()
        g_i, n_i = torch.nonzero(~same, as_tuple=True)
        if g_i.numel():                      # where they differ, the two centres are (nearly) equally far from the vector
            x = X[g_i, n_i]
            da = ((x - centres_in[g_i, got[g_i, n_i]]) ** 2).sum(-1)
            db = ((x - centres_in[g_i, codes_o[g_i, n_i]]) ** 2).sum(-1)
            assert bool(((da - db).abs() <= 1e-3 * torch.maximum(da, db) + 1e-5).all())
        agree = torch.ones(b, k, dtype=torch.bool)
        for gi in range(b):
            bad = torch.cat([got[gi][~same[gi]], codes_o[gi][~same[gi]]])
            agree[gi, bad] = False
        assert agree.float().mean().item() > 0.9
        assert torch.allclose(centres.cpu()[agree], cent_o.float()[agree], rtol=1e-4, atol=1e-4)
        centres_in = cent_o.float()


def _rows_membership(plan, n_keys, device):
    member = torch.zeros((plan.n_rows, n_keys), dtype=torch.bool, device=device)
    cnt = plan.cnt.long()
    cols = plan.cols.long()
    valid = torch.arange(cols.shape[1], device=device).unsqueeze(0) < cnt.unsqueeze(1)
    member.scatter_(1, torch.where(valid, cols, cols[:, :1]), True)   # a row's first entry stands in for its unused slots
    return member.cpu()


def test_config1_closed_form_plan_matches_the_oracle(cuda):
    """Headline configuration 1 at its full shape (batch 1, 32 query / 8 KV heads, 4096 keys, fp32, Sink 128 + Local 256)
    through the decode plan: ONE launch of the attention kernel with the sink + local columns in closed form,
    against the oracle directly, 1e-5."""
    from sparse_attention_hub_amd import _native as N

    sa = _sa()
    B, Hq, Hkv, Lk, D = 1, 32, 8, 4096, 128
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, torch.float32, seed=0)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=128), sa.LocalMaskerConfig(window_size=256)]))
    ra.return_attention_weights = False
    N.timing_enable(True)
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data={}, layer_idx=0)
    torch.cuda.synchronize()
    launches = N.timing_collect()
    N.timing_enable(False)
    assert w is None and set(launches) == {"k_sparse_attn"} and launches["k_sparse_attn"][0] == 1, launches
    plan = next(iter(ra._plans.values()))
    assert plan.att.closed_form == 1 and plan.att.closed_sink == 128 and plan.att.closed_window == 256
    oo, _, _ = O.research_attention([("sink", 128), ("local", 256)], q, k, v, None, D ** -0.5)
    assert rel_err(out, oo) < 1e-5


def test_config2_oracle_plan_at_full_shape_matches_the_oracle(cuda):
    """Headline configuration 2 at its full shape (batch 4, 32768 keys, bf16 with outlier channels, Sink 128 + Local 512 +
    OracleTopK 5 %) through the decode plan (scoring pass, selection that also writes the sink / local columns,
    attention), batch rows 0 and 3 against the oracle directly."""
    sa = _sa()
    B, Hq, Hkv, Lk, D = 4, 32, 8, 32768, 128
    sink, window, heavy = 128, 512, 1638
    dtype = torch.bfloat16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, outliers=True, seed=71)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[
        sa.SinkMaskerConfig(sink_size=sink), sa.LocalMaskerConfig(window_size=window), sa.OracleTopKConfig(heavy_size=heavy)]))
    ra.return_attention_weights = False
    out, _ = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data={}, layer_idx=0)
    torch.cuda.synchronize()
    plan = next(iter(ra._plans.values()))
    assert plan.kind == "oracle" and plan.att.Lk == Lk
    total = sink + window + heavy
    assert bool((plan.cnt.cpu() == total).all())
    member = _rows_membership(plan, Lk, cuda).view(B, Hq, Lk)
    specs = [("sink", sink), ("local", window), ("oracle_topk", heavy)]
    for b in (0, B - 1):
        oo, _, om = O.research_attention(specs, q[b:b + 1], k[b:b + 1], v[b:b + 1], None, D ** -0.5)
        want = om.to_dense()[0, :, 0] != 0
        # bf16 rounding of an fp32 accumulation: torch's CPU matmul may round a score on a rounding boundary the other
        # way, which can swap two neighbours at the threshold
        overlap = (member[b] & want).sum().item() / want.sum().item()
        assert overlap >= 0.999, (b, overlap)
        assert rel_err(out[b], oo[0]) < 2e-2


def test_config4_pq_plan_at_full_shape_matches_the_oracle(cuda):
    """Headline configuration 4 at its full shape (batch 4, 32768 keys, bf16 with outlier channels, Sink 128 + Local 256 +
    PQCache top-1024 with 16 sub-vectors of 8 and 256 centres; 3 Lloyd iterations here): the warm step through the
    decode plan (ADC scoring, selection that also writes the sink / local columns, attention), batch rows 0 and 3
    against the oracle given the kernel's codebook: selected sets bit-exact."""
    sa = _sa()
    B, Hq, Hkv, Lk, D = 4, 32, 8, 32768, 128
    sink, window, heavy = 128, 256, 1024
    dtype = torch.bfloat16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, outliers=True, seed=73)
    q0 = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=74)[0]
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[
        sa.SinkMaskerConfig(sink_size=sink), sa.LocalMaskerConfig(window_size=window),
        sa.PQCacheConfig(heavy_size=heavy, pq_group_factor=16, pq_bits=8, kmeans_iter=3, init_offset=sink, metric="euclidean")]))
    ra.return_attention_weights = False
    meta = {}
    kc, vc = k.to(cuda), v.to(cuda)
    ra.custom_attention(None, q0.to(cuda), kc[:, :, :Lk - 1], vc[:, :, :Lk - 1], None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    out, _ = ra.custom_attention(None, q.to(cuda), kc, vc, None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    torch.cuda.synchronize()
    plan = next(iter(ra._plans.values()))
    assert plan.kind == "pq" and plan.att.Lk == Lk
    total = sink + window + heavy
    assert bool((plan.cnt.cpu() == total).all())
    member = _rows_membership(plan, Lk, cuda).view(B, Hq, Lk)
    book = meta["pq_codebook"][0]
    assert book.n == Lk - 1 - sink               # the newest key sits inside the local window: quantised with the next block
    for b in (0, B - 1):
        cent = meta["pq_centroids"][0][b:b + 1].cpu()
        codes = book.to_reference()[b:b + 1].cpu()
        # the oracle scores every quantised key; the newest one is not quantised yet and lies inside the local window
        kb, vb = k[b:b + 1], v[b:b + 1]
        codes_full = torch.cat([codes, codes[:, -1:]], dim=1)        # a stand-in code for the window key (already active)
        oo, _, om = O.research_attention([("sink", sink), ("local", window), ("pq_topk", heavy, sink, cent, codes_full)],
                                         q[b:b + 1], kb, vb, None, D ** -0.5)
        assert torch.equal(member[b], om.to_dense()[0, :, 0] != 0), f"batch row {b}: selected sets differ"
        assert rel_err(out[b], oo[0]) < 2e-2


@pytest.mark.parametrize("B", [4, 16])
def test_config3_chain_at_other_batch_sizes_matches_the_oracle(cuda, B):
    """The HashAttention decode step of configuration 3 at batch 4 (128 mask rows: fewer rows than CUs) and batch 16
    (512 rows: two rounds of one workgroup per CU), 32768 keys: first and last batch row against the oracle given the
    kernel's signatures, selected sets bit-exact."""
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    sa = _sa()
    Hq, Hkv, Lk, D = 32, 8, 32768, 128
    sink, window, heavy = 128, 512, 2048
    dtype = torch.bfloat16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=81)
    q0 = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=82)[0]
    wts = random_hat_weights(1, Hq, D, 32, 3, 128, dtype=dtype, seed=1)
    cfg = sa.HashAttentionTopKMaskerConfig(heavy_size=heavy, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                           hat_mlp_activation="silu", hat_weights=wts)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=sink), sa.LocalMaskerConfig(window_size=window), cfg]))
    ra.return_attention_weights = False
    meta = {}
    kc, vc = k.to(cuda), v.to(cuda)
    scaling = D ** -0.5
    for n in (Lk - 2, Lk - 1):
        ra.custom_attention(None, q0.to(cuda), kc[:, :, :n], vc[:, :, :n], None, scaling, 0.0, sparse_meta_data=meta, layer_idx=0)
    out, _ = ra.custom_attention(None, q.to(cuda), kc, vc, None, scaling, 0.0, sparse_meta_data=meta, layer_idx=0)
    torch.cuda.synchronize()
    plan = next(iter(ra._plans.values()))
    total = sink + window + heavy
    assert plan.kind == "hash" and bool((plan.cnt.cpu() == total).all())
    member = _rows_membership(plan, Lk, cuda).view(B, Hq, Lk)
    cache = meta["key"][0]
    qcodes = torch.empty((B * Hq, 2), dtype=torch.int32, device=cuda)
    ra.maskers[2]._hash(q.to(cuda), Hq, Hq, 0, 1, 0, "query", qcodes, 1, 0)
    qsig = _unpack_codes(qcodes).view(B, Hq, 1, 32)
    specs = [("sink", sink), ("local", window), ("hash_topk", heavy, wts[0], "silu")]
    for b in (0, B - 1):
        state = {"key_sig": _unpack_codes(cache.codes[b:b + 1, :, :cache.n]), "query_sig": qsig[b:b + 1]}
        oo, _, om = O.research_attention(specs, q[b:b + 1], k[b:b + 1], v[b:b + 1], None, scaling, state=state)
        assert torch.equal(member[b], om.to_dense()[0, :, 0] != 0), f"batch row {b}: selected sets differ"
        assert rel_err(out[b], oo[0]) < 2e-2


@pytest.mark.parametrize("kind", ["hash", "oracle", "pq"])
def test_rows_shared_by_several_workgroups_give_the_same_bits_every_time(cuda, kind):
    """Batch 1 at 32768 keys: 32 mask rows, 8 workgroups per row, the one that arrives last merges. The order of arrival
    changes from launch to launch, the result must not: 40 repetitions of the same decode step (same queries, same keys)
    through the plan give the same output bits and the same rows, and the arrival counters are back at zero after each."""
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    sa = _sa()
    B, Hq, Hkv, Lk, D = 1, 32, 8, 32768, 128
    sink, window, heavy = 128, 256, 1024
    dtype = torch.bfloat16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=91, outliers=(kind != "hash"), device=cuda)
    if kind == "hash":
        wts = random_hat_weights(1, Hq, D, 32, 3, 128, dtype=dtype, seed=1)
        top = sa.HashAttentionTopKMaskerConfig(heavy_size=heavy, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                               hat_mlp_activation="silu", hat_weights=wts)
    elif kind == "oracle":
        top = sa.OracleTopKConfig(heavy_size=heavy)
    else:
        top = sa.PQCacheConfig(heavy_size=heavy, pq_group_factor=16, pq_bits=8, kmeans_iter=2, init_offset=sink, metric="euclidean")
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=sink), sa.LocalMaskerConfig(window_size=window), top]))
    ra.return_attention_weights = False
    meta = {}
    scaling = D ** -0.5
    # the caches are built on the first call (one key short), the plan takes over from the second
    ra.custom_attention(None, q, k[:, :, :Lk - 1], v[:, :, :Lk - 1], None, scaling, 0.0, sparse_meta_data=meta, layer_idx=0)
    first, first_rows = None, None
    for rep in range(40):
        out, _ = ra.custom_attention(None, q, k, v, None, scaling, 0.0, sparse_meta_data=meta, layer_idx=0)
        plan = next(iter(ra._plans.values()))
        torch.cuda.synchronize()
        assert int(plan.tickets.abs().max()) == 0, rep
        rows = torch.sort(plan.cols[:, :sink + window + heavy], dim=1).values
        if first is None:
            first, first_rows = out.clone(), rows.clone()
            assert plan.kind == kind and bool((plan.cnt == sink + window + heavy).all())
            assert bool(torch.isfinite(out.float()).all()) and float(out.float().abs().max()) > 0
        else:
            assert torch.equal(out, first), f"repetition {rep}: output bits differ"
            assert torch.equal(rows, first_rows), f"repetition {rep}: rows differ"
