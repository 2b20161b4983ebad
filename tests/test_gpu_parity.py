"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle on the same
seeded inputs. Bars: index sets bit-exact (ties to the lowest column); attention outputs
within 1e-5 relative error for fp32 and 2e-2 for bf16."""
import copy
import ctypes as C
import math

import pytest
import torch

from _util import make_qkv, rel_err
from oracle import reference_path as O

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def _sa():
    import sparse_attention_hub_amd.sparse_attention as sa

    return sa


def _same_output(o_plan, o_ref, n_rows):
    """Plan against masker-by-masker path. With at least as many rows as the one-workgroup-per-row forms need, both sum in
    the same order: bit-identical. With fewer rows the one-kernel forms give a row several workgroups, which deal the
    row's entries out differently: the same columns, sums that may differ in a last bit."""
    if n_rows >= 192:
        return torch.equal(o_plan, o_ref)
    return rel_err(o_plan, o_ref) < 4e-3


def _run_chain(cuda, cfgs, specs, B, Hq, Hkv, Lq, Lk, D, dtype, amask=None, sinks=None, outliers=False, seed=0,
               meta=None, check_weights=True):
    sa = _sa()
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, dtype, seed=seed, outliers=outliers)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    scaling = D ** -0.5
    meta = {} if meta is None else meta
    kw = dict(sparse_meta_data=meta, layer_idx=0)
    if sinks is not None:
        kw["s_aux"] = sinks.to(cuda)
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None if amask is None else amask.to(cuda),
                                 scaling, 0.0, **kw)
    torch.cuda.synchronize()
    oo, ow, om = O.research_attention(specs, q, k, v, amask, scaling, sinks)
    assert out.shape == oo.shape and out.dtype == dtype
    err = rel_err(out, oo)
    assert err < TOL[dtype], f"output rel err {err}"
    if check_weights:
        assert w.shape == ow.shape
        if om.kind == "dense":
            assert torch.equal(w.cpu() != 0, ow != 0)
        assert (w.float().cpu() - ow.float()).abs().max().item() < (1e-6 if dtype == torch.float32 else 1e-2)
    return out, w, om, meta


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [16, 64, 128])
def test_sink_local_chain(cuda, dtype, D):
    sa = _sa()
    _run_chain(cuda, [sa.SinkMaskerConfig(sink_size=4), sa.LocalMaskerConfig(window_size=8)],
               [("sink", 4), ("local", 8)], 2, 4, 2, 1, 333, D, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [8, 24, 80, 96, 112, 160, 256])
def test_head_dims_that_are_not_16_32_64_128(cuda, dtype, D):
    """The reference's masked attention takes any head_dim (utils/mask_attention_utils.py:406-491); the kernels pad a
    head_dim that is a multiple of 8 up to 256 to the next power of two: Sink + Local rows (whole-row form), dense
    attention with sink logits (split form and merge kernel), and - up to 128 - the OracleTopK scoring pass."""
    sa = _sa()
    _run_chain(cuda, [sa.SinkMaskerConfig(sink_size=4), sa.LocalMaskerConfig(window_size=8)],
               [("sink", 4), ("local", 8)], 2, 4, 2, 1, 333, D, dtype)
    _run_chain(cuda, [], [], 1, 4, 2, 2, 1500, D, dtype, sinks=torch.tensor([0.1, -0.3, 0.5, 1.0]))
    if D <= 128:
        _run_chain(cuda, [sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=32), sa.OracleTopKConfig(heavy_size=40)],
                   [("sink", 16), ("local", 32), ("oracle_topk", 40)], 2, 8, 2, 1, 900, D, dtype)
    else:
        with pytest.raises(ValueError, match="head_dim"):
            _run_chain(cuda, [sa.OracleTopKConfig(heavy_size=40)], [("oracle_topk", 40)], 1, 4, 2, 1, 300, D, dtype)


def test_sink_local_index_form_is_bit_exact(cuda):
    sa = _sa()
    B, Hq, Lq, Lk = 2, 4, 3, 70
    q, k, v = make_qkv(B, Hq, 2, Lq, Lk, 16, torch.float32)
    m = sa.Mask.create_empty_mask((B, Hq, Lq, Lk), torch.float32, cuda)
    for cfg in (sa.SinkMaskerConfig(sink_size=5), sa.LocalMaskerConfig(window_size=9)):
        m = sa.ResearchMasker.create_masker_from_config(cfg).add_mask(
            keys=k.to(cuda), queries=q.to(cuda), values=v.to(cuda), attention_mask=None, scaling=1.0, dropout=0.0,
            sparse_meta_data={}, previous_mask=m)
    om = O.local(O.sink(O.OMask.empty((B, Hq, Lq, Lk), torch.float32), 5), 9)
    idx, ptr, data = m.get_index_mask()
    oidx, optr, odata = om.index_form()
    assert idx.dtype == torch.int64 and ptr.dtype == torch.int64
    assert torch.equal(idx.cpu(), oidx) and torch.equal(ptr.cpu(), optr) and torch.equal(data.cpu(), odata)
    assert torch.equal(m.get_dense_mask().cpu(), om.to_dense())


def test_local_merges_into_dense_previous_and_clears_future(cuda):
    # reference pattern: previous [0,1] + local window 2 on Lq=3, Lk=8 (test_basic_fixed.py:299-312)
    sa = _sa()
    prev = torch.zeros(1, 1, 3, 8)
    prev[..., :2] = 1.0
    prev[..., 0, 7] = 1.0   # a future column of query 0: must be cleared
    pm = sa.Mask.create_mask_from_dense_mask((1, 1, 3, 8), prev.to(cuda), torch.float32)
    q, k, v = make_qkv(1, 1, 1, 3, 8, 16, torch.float32)
    m = sa.LocalMasker(sa.LocalMaskerConfig(window_size=2)).add_mask(
        keys=k.to(cuda), queries=q.to(cuda), values=v.to(cuda), attention_mask=None, scaling=1.0, dropout=0.0,
        sparse_meta_data={}, previous_mask=pm)
    want = torch.tensor([[1, 1, 0, 0, 1, 1, 0, 0], [1, 1, 0, 0, 0, 1, 1, 0], [1, 1, 0, 0, 0, 0, 1, 1]], dtype=torch.float32)
    assert torch.equal(m.get_dense_mask()[0, 0].cpu(), want)


def test_full_mask_shortcuts(cuda):
    sa = _sa()
    q, k, v = make_qkv(1, 2, 1, 1, 8, 16, torch.float32)
    args = dict(keys=k.to(cuda), queries=q.to(cuda), values=v.to(cuda), attention_mask=None, scaling=1.0, dropout=0.0,
                sparse_meta_data={})
    e = sa.Mask.create_empty_mask((1, 2, 1, 8), torch.float32, cuda)
    assert sa.SinkMasker(sa.SinkMaskerConfig(sink_size=8)).add_mask(previous_mask=e, **args).is_full_mask()
    assert sa.LocalMasker(sa.LocalMaskerConfig(window_size=7)).add_mask(previous_mask=e, **args).is_full_mask()
    assert sa.OracleTopK(sa.OracleTopKConfig(heavy_size=8)).add_mask(previous_mask=e, **args).is_full_mask()
    f = sa.Mask.create_full_mask((1, 2, 1, 8), torch.float32, cuda)
    assert sa.SinkMasker(sa.SinkMaskerConfig(sink_size=2)).add_mask(previous_mask=f, **args) is f


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_attention_with_sinks_and_additive_mask(cuda, dtype):
    B, Hq, Hkv, Lq, Lk, D = 2, 4, 2, 2, 700, 64
    am = torch.zeros(B, 1, Lq, Lk)
    am[0, :, :, -50:] = torch.finfo(torch.float32).min
    am = am.to(dtype)
    _run_chain(cuda, [], [], B, Hq, Hkv, Lq, Lk, D, dtype, amask=am, sinks=torch.tensor([0.1, -0.3, 0.5, 1.0]))


@pytest.mark.parametrize("dtype,D,Lk,heavy", [(torch.float32, 32, 1000, 50), (torch.bfloat16, 128, 4096, 0.05),
                                              (torch.bfloat16, 64, 777, 33), (torch.float32, 128, 5000, 0.02)])
def test_oracle_topk_chain(cuda, dtype, D, Lk, heavy):
    sa = _sa()
    _run_chain(cuda, [sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=32), sa.OracleTopKConfig(heavy_size=heavy)],
               [("sink", 16), ("local", 32), ("oracle_topk", heavy)], 2, 8, 2, 1, Lk, D, dtype, outliers=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_training_mode_dropout_follows_the_oracle_stream(cuda, dtype):
    """Attention dropout in training mode (mask_attention_utils.py:234-238: torch.nn.functional.dropout on the exp
    weights): the kernels draw an entry's fate from Philox keyed by torch's seed and a per-call offset, the oracle
    draws the same stream, so outputs and dense probabilities agree entry by entry, with a sparse mask, a sink logit
    and the dense path; eval mode and p = 0 leave everything as it was; p >= 1 is refused."""
    from sparse_attention_hub_amd.sparse_attention.utils import mask_attention_utils as mau

    sa = _sa()
    B, Hq, Hkv, Lq, Lk, D, p = 2, 4, 2, 1, 600, 64, 0.25
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, dtype, seed=9)
    sinks = torch.tensor([0.2, -0.1, 0.4, 0.0])
    cfgs = [sa.SinkMaskerConfig(sink_size=8), sa.LocalMaskerConfig(window_size=16), sa.OracleTopKConfig(heavy_size=100)]
    specs = [("sink", 8), ("local", 16), ("oracle_topk", 100)]
    train, evalm = torch.nn.Module(), torch.nn.Module()
    train.train()
    evalm.eval()
    torch.manual_seed(1234)
    seed = torch.initial_seed()
    # the per-call offsets are draws from torch's default generator: the same numbers a generator seeded alike gives
    expect = torch.Generator().manual_seed(1234)
    tol_w = 1e-6 if dtype == torch.float32 else 1e-2
    outs = []
    for call, (c, sp) in enumerate(((cfgs, specs), (cfgs, specs), ([], []))):    # the third: dense attention
        offset = int(torch.randint(0, 2 ** 62, (1,), dtype=torch.int64, generator=expect).item())
        ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=c))
        out, w = ra.custom_attention(train, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, p, sparse_meta_data={},
                                     layer_idx=0, s_aux=sinks.to(cuda))
        oo, ow, _ = O.research_attention(sp, q, k, v, None, D ** -0.5, sinks, dropout=(p, seed, offset))
        assert rel_err(out, oo) < TOL[dtype], call
        assert torch.equal(w.cpu() != 0, ow != 0), call                        # the same entries survive
        assert (w.float().cpu() - ow.float()).abs().max().item() < tol_w
        outs.append(out)
    # re-seeding reproduces the dropout masks (as torch's generator does for the reference)
    torch.manual_seed(1234)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    again, _ = ra.custom_attention(train, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, p, sparse_meta_data={},
                                   layer_idx=0, s_aux=sinks.to(cuda))
    assert torch.equal(again, outs[0])
    expect = torch.Generator().manual_seed(1234)
    torch.randint(0, 2 ** 62, (1,), dtype=torch.int64, generator=expect)         # the draw of the call above
    # the "true" dense attention of the error metric: dropout of the normalised probabilities (SDPA with dropout_p on
    # the reference's dense path, mask_attention_utils.py:40-52): the denominator keeps the dropped entries
    offset = int(torch.randint(0, 2 ** 62, (1,), dtype=torch.int64, generator=expect).item())
    true_out, _ = mau.get_true_attention_output(train, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, p)
    empty = O.OMask.empty((B, Hq, Lq, Lk), dtype)
    want, _ = O.masked_attention(q, k, v, None, None, D ** -0.5, empty, dropout=(p, seed, offset), dropout_numerator_only=True)
    assert rel_err(true_out, want) < TOL[dtype]
    both, _ = O.masked_attention(q, k, v, None, None, D ** -0.5, empty, dropout=(p, seed, offset))
    assert rel_err(true_out, both) > 10 * TOL[dtype] or dtype == torch.bfloat16   # and it is not the other form
    assert not torch.equal(outs[0], outs[1])                                     # every call draws anew
    # about a quarter of the entries of a row are gone
    kept = float((w != 0).float().mean())
    assert abs(kept - (1 - p)) < 0.05
    # eval mode: no dropout, whatever p is; and the fast decode plan is free to run again
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    out_e, _ = ra.custom_attention(evalm, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, p, sparse_meta_data={}, layer_idx=0)
    oo, _, _ = O.research_attention(specs, q, k, v, None, D ** -0.5)
    assert rel_err(out_e, oo) < TOL[dtype]
    with pytest.raises(ValueError):
        ra.custom_attention(train, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 1.0, sparse_meta_data={}, layer_idx=0)


def test_oracle_topk_many_ties_lowest_index(cuda):
    # integer-valued keys => heavy ties at the threshold; the selected set must be the lowest columns
    sa = _sa()
    g = torch.Generator().manual_seed(0)
    B, Hq, Hkv, Lk, D = 1, 2, 1, 3000, 16
    q = torch.zeros(B, Hq, 1, D)
    q[..., 0] = 1.0
    k = torch.zeros(B, Hkv, Lk, D)
    k[..., 0] = torch.randint(-3, 4, (B, Hkv, Lk), generator=g).float()
    v = torch.randn(B, Hkv, Lk, D, generator=g)
    for dtype in (torch.float32, torch.bfloat16):
        ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
            masker_configs=[sa.SinkMaskerConfig(sink_size=3), sa.OracleTopKConfig(heavy_size=500)]))
        out, w = ra.custom_attention(None, q.to(dtype).to(cuda), k.to(dtype).to(cuda), v.to(dtype).to(cuda), None, 0.25, 0.0,
                                     sparse_meta_data={})
        _, ow, om = O.research_attention([("sink", 3), ("oracle_topk", 500)], q.to(dtype), k.to(dtype), v.to(dtype), None, 0.25)
        assert torch.equal(w.cpu() != 0, om.to_dense() != 0)


def _hat(sa, Hq, D, dtype, hidden=32, bits=32, seed=1):
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    return random_hat_weights(1, Hq, D, bits, 3, hidden, dtype=dtype, seed=seed)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("use_amask", [False, True])
def test_hash_topk_chain(cuda, dtype, use_amask):
    """Selection + attention are bit-exact / in tolerance *given the signatures*: the oracle scores
    the kernel's own codes (unpacked to the reference's +-1/0 floats), so MLP rounding noise
    (tested separately below) cannot move a key across the top-k threshold."""
    sa = _sa()
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.hashattention_top_k import (
        HashAttentionTopKMasker,
    )

    B, Hq, Hkv, Lk, D = 2, 8, 2, 1500, 128
    wts = _hat(sa, Hq, D, dtype, hidden=128)
    cfg = sa.HashAttentionTopKMaskerConfig(heavy_size=128, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                           hat_mlp_activation="silu", hat_weights=wts)
    am = None
    if use_amask:
        am = torch.zeros(B, 1, 1, Lk)
        am[1, :, :, 100:400] = torch.finfo(torch.float32).min
        am = am.to(dtype)
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=64), cfg]))
    meta = {}
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None if am is None else am.to(cuda),
                                 D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    ksig = meta["key"][0].unpack(torch.float32).cpu()
    masker = HashAttentionTopKMasker(cfg)
    qcodes = torch.empty((B * Hq, 2), dtype=torch.int32, device=cuda)
    masker._hash(q.to(cuda), Hq, Hq, 0, 1, 0, "query", qcodes, 1, 0)
    qc = qcodes.cpu().to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(32)
    qsig = ((((qc[:, 0:1] >> shifts) & 1) * 2 - 1) * ((qc[:, 1:2] >> shifts) & 1)).float().view(B, Hq, 1, 32)
    state = {"key_sig": ksig, "query_sig": qsig}
    oo, ow, om = O.research_attention([("sink", 16), ("local", 64), ("hash_topk", 128, wts[0], "silu")], q, k, v, am,
                                      D ** -0.5, state=state)
    assert torch.equal(w.cpu() != 0, om.to_dense() != 0)            # index sets: bit-exact
    assert torch.all((om.to_dense() != 0).sum(-1) == 16 + 64 + 128)
    assert rel_err(out, oo) < TOL[dtype]
    # and the signatures themselves agree with the float MLP almost everywhere
    sig = O.hash_signatures(O.repeat_kv(k, Hq // Hkv), wts[0]["key_matrix"], wts[0]["key_bias"], "silu")
    assert (ksig == sig.float()).float().mean().item() >= 0.9995


def test_hash_masker_from_weight_file_matches_in_memory_weights(cuda, tmp_path):
    """`hat_weight_file=` (the reference's pickle layout, hashattention_utils.py:155-180) through the kernels:
    same codes, same selected sets, same output bits as `hat_weights=` with the tensors it was written from."""
    import pickle

    sa = _sa()
    B, Hq, Hkv, Lk, D = 2, 8, 2, 900, 128
    dtype = torch.bfloat16
    wts = _hat(sa, Hq, D, dtype, hidden=128)
    path = tmp_path / "hat_weights.pkl"
    with open(path, "wb") as f:
        pickle.dump(wts, f)
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=12)
    results = []
    for source in (dict(hat_weights=wts), dict(hat_weight_file=str(path))):
        cfg = sa.HashAttentionTopKMaskerConfig(heavy_size=96, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                               hat_mlp_activation="silu", **source)
        ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
            masker_configs=[sa.SinkMaskerConfig(sink_size=8), sa.LocalMaskerConfig(window_size=32), cfg]))
        meta = {}
        out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0,
                                     sparse_meta_data=meta, layer_idx=0)
        results.append((out.cpu(), w.cpu(), meta["key"][0].unpack(torch.float32).cpu()))
    (o1, w1, s1), (o2, w2, s2) = results
    assert torch.equal(s1, s2) and torch.equal(w1, w2) and torch.equal(o1, o2)
    assert torch.all((w1 != 0).sum(-1) == 8 + 32 + 96)
    with pytest.raises(ValueError):
        sa.ResearchMasker.create_masker_from_config(sa.HashAttentionTopKMaskerConfig(
            heavy_size=96, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128, hat_mlp_activation="silu",
            hat_weights=wts, hat_weight_file=str(path)))


def test_hash_signatures_bits_and_cache_growth(cuda):
    sa = _sa()
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.hashattention_top_k import (
        HashAttentionTopKMasker,
    )

    for dtype in (torch.float32, torch.bfloat16):
        B, Hq, Hkv, Lk, D = 1, 4, 2, 300, 64
        wts = _hat(sa, Hq, D, dtype, hidden=48, bits=24)
        cfg = sa.HashAttentionTopKMaskerConfig(heavy_size=8, hat_bits=24, hat_mlp_layers=3, hat_mlp_hidden_size=48,
                                               hat_mlp_activation="gelu", hat_weights=wts)
        masker = HashAttentionTopKMasker(cfg)
        _, k, _ = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype)
        meta = {}
        kc = k.to(cuda)
        masker._update_key_signatures(kc[:, :, :200].contiguous(), Hq, meta, 0)
        cache = masker._update_key_signatures(kc, Hq, meta, 0)          # only keys 200.. are hashed now
        assert cache.shape == (B, Hq, Lk, 24)
        sig = O.hash_signatures(O.repeat_kv(k, 2), wts[0]["key_matrix"], wts[0]["key_bias"], "gelu")
        got = cache.unpack(torch.float32).cpu()
        agree = (got == sig.float()).float().mean().item()
        # accumulation order differs from torch's: a value within rounding noise of 0 (or, in bf16, of a
        # rounding boundary of an intermediate activation) may land on the other side
        assert agree >= 0.9995, agree
        with pytest.raises(ValueError, match="less than cached"):
            masker._update_key_signatures(kc[:, :, :100].contiguous(), Hq, meta, 0)


# (head_dim, sub-spaces, bits). 16 one-byte codes = one 16-byte load; (128, 2 | 4) with 4 / 6 / 8 bits are the geometries
# the reference's own PQCache configurations use (sub-vectors of 64 and 32: docs/baselines/pqcache.md:17-25,
# benchmark/raytune/config_builders/pqcache.py:51-67); 256 centres of 64 dimensions take their sums in a launch of their own
@pytest.mark.parametrize("geometry", [(64, 8, 4), (128, 16, 4), (128, 2, 6), (128, 4, 6), (128, 4, 4), (128, 2, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pq_chain_cold_and_warm(cuda, dtype, geometry):
    sa = _sa()
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.utils.pq_utils import (
        gather_sub_vectors, seeded_initial_centres,
    )

    D, n_sub, bits = geometry
    B, Hq, Hkv, Lk = 2, 8, 2, 1200
    off, iters, heavy = 16, 5, 64
    n_cent = 2 ** bits
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, outliers=True)
    cfg = sa.PQCacheConfig(heavy_size=heavy, pq_group_factor=n_sub, pq_bits=bits, kmeans_iter=iters, init_offset=off,
                           metric="euclidean")
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=off), sa.LocalMaskerConfig(window_size=32), cfg]))
    meta = {}
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    # Lloyd parity from the same start (and the same reseed table)
    X = O.pq_split(k, off, n_sub)
    start = seeded_initial_centres(B * Hkv * n_sub, Lk - off, n_cent, 0, torch.device("cpu"))
    c0 = gather_sub_vectors(k, off, n_sub, start)
    reseed = torch.randint(0, Lk - off, (iters, B * Hkv * n_sub, n_cent), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    codes_o, cent_o = O.kmeans_lloyd(X, c0, iters, reseed_idx=reseed)
    book = meta["pq_codebook"][0]
    assert book.shape == (B, Lk - off, Hkv, n_sub)
    codes = book.to_reference().cpu()
    codes_o = codes_o.reshape(B, Hkv, n_sub, Lk - off).permute(0, 3, 1, 2)
    assert (codes == codes_o).float().mean().item() >= 0.999
    cent = meta["pq_centroids"][0]
    assert cent.dtype == dtype and cent.shape == (B, Hkv, n_sub, n_cent, D // n_sub)
    # centres: fp32 sums are accumulated with atomics (order differs); bf16 storage may land one ulp apart
    rtol = 1e-3 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(cent.float().cpu().reshape(-1), cent_o.float().reshape(-1), rtol=rtol, atol=1e-3)
    # scoring + top-k + attention given the kernel's own codebook
    oo, ow, om = O.research_attention([("sink", off), ("local", 32), ("pq_topk", heavy, off, cent.cpu(), codes)], q, k, v, None, D ** -0.5)
    assert rel_err(out, oo) < TOL[dtype]
    assert torch.equal(w.cpu() != 0, om.to_dense() != 0)
    # warm step: three appended keys are quantised against the frozen centroids
    q2, kn, vn = make_qkv(B, Hq, Hkv, 1, 3, D, dtype, seed=5)
    k2, v2 = torch.cat([k, kn], 2), torch.cat([v, vn], 2)
    out2, w2 = ra.custom_attention(None, q2.to(cuda), k2.to(cuda), v2.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    codes2 = meta["pq_codebook"][0].to_reference().cpu()
    assert torch.equal(codes2[:, : Lk - off], codes)
    assert torch.equal(codes2[:, Lk - off:], O.pq_quantize_new(kn, cent.cpu()))
    oo2, _, om2 = O.research_attention([("sink", off), ("local", 32), ("pq_topk", heavy, off, cent.cpu(), codes2)], q2, k2, v2, None, D ** -0.5)
    assert rel_err(out2, oo2) < TOL[dtype]
    assert torch.equal(w2.cpu() != 0, om2.to_dense() != 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pq_chain_inner_product_metric(cuda, dtype):
    """PQCache(metric="ip"): the keys are clustered with one extra coordinate sqrt(phi - ||x||^2) per
    sub-vector (pq_utils.py:585-612), later keys are quantised with a zero there (:615-640), and the
    scoring table ignores it (pq_top_k.py:457-458). Lloyd steps from the same start vectors against the
    oracle, then selection and attention given the kernel's own codebook, cold and warm."""
    sa = _sa()
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.utils.pq_utils import (
        seeded_initial_centres,
    )

    B, Hq, Hkv, Lk, D = 2, 8, 2, 1000, 64
    n_sub, bits, off, iters, heavy = 8, 4, 16, 4, 64
    n_cent, d = 2 ** bits, D // n_sub
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, outliers=True, seed=9)
    cfg = sa.PQCacheConfig(heavy_size=heavy, pq_group_factor=n_sub, pq_bits=bits, kmeans_iter=iters, init_offset=off, metric="ip")
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=off), sa.LocalMaskerConfig(window_size=32), cfg]))
    meta = {}
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    X, phi = O.pq_split_ip(k, off, n_sub)
    assert X.shape == (B * Hkv * n_sub, Lk - off, d + 1)
    assert torch.allclose(meta["pq_ip2l2_phi"][0].float().cpu(), phi.float(), rtol=2 ** -7)
    start = seeded_initial_centres(B * Hkv * n_sub, Lk - off, n_cent, 0, torch.device("cpu")).long()
    c0 = torch.gather(X.float(), 1, start.unsqueeze(-1).expand(-1, -1, d + 1))
    reseed = torch.randint(0, Lk - off, (iters, B * Hkv * n_sub, n_cent), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    codes_o, cent_o = O.kmeans_lloyd(X, c0, iters, reseed_idx=reseed)
    codes = meta["pq_codebook"][0].to_reference().cpu()
    codes_o = codes_o.reshape(B, Hkv, n_sub, Lk - off).permute(0, 3, 1, 2)
    # the extra coordinate is computed in the key dtype on both sides; in bf16 a device-side sum may round it
    # differently for a few vectors, which can move them to a neighbouring centre
    assert (codes == codes_o).float().mean().item() >= (0.999 if dtype == torch.float32 else 0.98)
    cent = meta["pq_centroids"][0]
    assert cent.dtype == dtype and cent.shape == (B, Hkv, n_sub, n_cent, d + 1)
    if dtype == torch.float32:
        assert torch.allclose(cent.cpu().reshape(-1), cent_o.reshape(-1), rtol=1e-3, atol=1e-3)
    oo, ow, om = O.research_attention([("sink", off), ("local", 32), ("pq_topk", heavy, off, cent.cpu(), codes)], q, k, v, None, D ** -0.5)
    assert rel_err(out, oo) < TOL[dtype]
    assert torch.equal(w.cpu() != 0, om.to_dense() != 0)
    q2, kn, vn = make_qkv(B, Hq, Hkv, 1, 3, D, dtype, seed=6)
    k2, v2 = torch.cat([k, kn], 2), torch.cat([v, vn], 2)
    out2, w2 = ra.custom_attention(None, q2.to(cuda), k2.to(cuda), v2.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data=meta, layer_idx=0)
    codes2 = meta["pq_codebook"][0].to_reference().cpu()
    assert torch.equal(codes2[:, : Lk - off], codes)
    assert torch.equal(codes2[:, Lk - off:], O.pq_quantize_new(kn, cent.cpu()))
    oo2, _, om2 = O.research_attention([("sink", off), ("local", 32), ("pq_topk", heavy, off, cent.cpu(), codes2)], q2, k2, v2, None, D ** -0.5)
    assert rel_err(out2, oo2) < TOL[dtype]
    assert torch.equal(w2.cpu() != 0, om2.to_dense() != 0)


def test_rows_from_dense_round_trip_with_weights(cuda):
    sa = _sa()
    g = torch.Generator().manual_seed(3)
    dense = (torch.rand(3, 5, 2, 300, generator=g) > 0.8).float() * (torch.rand(3, 5, 2, 300, generator=g) * 0.5 + 0.5)
    m = sa.Mask.create_mask_from_dense_mask(dense.shape, dense.to(cuda), torch.float32)
    rows = m.to_rows(0)
    back = sa.Mask.create_mask_from_rows(dense.shape, rows, torch.float32)
    assert torch.equal(back.get_dense_mask().cpu(), dense)
    idx, ptr, data = back.get_index_mask()
    oidx, optr, odata = O.OMask("dense", tuple(dense.shape), torch.float32, dense).index_form()
    assert torch.equal(idx.cpu(), oidx) and torch.equal(ptr.cpu(), optr) and torch.equal(data.cpu(), odata)


def test_weighted_mask_attention(cuda):
    # inverse-weight semantics exp/(w + 1e-6) incl. bf16 evaluation of the reciprocal
    sa = _sa()
    from sparse_attention_hub_amd.sparse_attention.utils.mask_attention_utils import get_masked_attention_output

    for dtype in (torch.float32, torch.bfloat16):
        B, Hq, Hkv, Lk, D = 1, 4, 2, 500, 64
        q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=2)
        g = torch.Generator().manual_seed(4)
        dm = ((torch.rand(B, Hq, 1, Lk, generator=g) > 0.7).float() * torch.rand(B, Hq, 1, Lk, generator=g)).to(dtype)
        dm[..., :4] = 1.0
        mask = sa.Mask.create_mask_from_dense_mask(dm.shape, dm.to(cuda), dtype)
        out, w = get_masked_attention_output(None, q.to(cuda), k.to(cuda), v.to(cuda), None, None, D ** -0.5, 0.0, mask,
                                             return_attention_weights=True)
        oo, ow = O.masked_attention(q, k, v, None, None, D ** -0.5, O.OMask("dense", tuple(dm.shape), dtype, dm))
        assert rel_err(out, oo) < TOL[dtype]
        assert torch.equal(w.cpu() != 0, ow != 0)


def test_missing_sparse_meta_data_and_layer_idx_raise(cuda):
    sa = _sa()
    q, k, v = make_qkv(1, 2, 1, 1, 64, 16, torch.float32)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[]))
    with pytest.raises(ValueError, match="sparse_meta_data must be provided"):
        ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, 1.0, 0.0)
    wts = _hat(sa, 2, 16, torch.float32)
    cfg = sa.HashAttentionTopKMaskerConfig(heavy_size=4, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=32,
                                           hat_mlp_activation="silu", hat_weights=wts)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[cfg]))
    with pytest.raises(ValueError, match="layer_idx must be provided"):
        ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, 1.0, 0.0, sparse_meta_data={})


@pytest.mark.parametrize("kind", ["fixed", "hash", "oracle", "pq", "pq_wide"])
def test_decode_plan_matches_masker_by_masker_path(cuda, kind):
    """The one-call decode plan (weights not requested) gives bit-identical outputs to the general
    masker-by-masker path over several appended-key steps, and really is the path taken."""
    sa = _sa()
    dtype = torch.bfloat16
    B, Hq, Hkv, Lk, D = 2, 8, 2, 2000, 128
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk + 4, D, dtype, outliers=True)
    cfgs = [sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=64)]
    if kind == "hash":
        cfgs.append(sa.HashAttentionTopKMaskerConfig(heavy_size=100, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                                     hat_mlp_activation="silu", hat_weights=_hat(sa, Hq, D, dtype, hidden=128)))
    elif kind == "oracle":
        cfgs.append(sa.OracleTopKConfig(heavy_size=0.05))
    elif kind == "pq":
        cfgs.append(sa.PQCacheConfig(heavy_size=64, pq_group_factor=16, pq_bits=6, kmeans_iter=4, init_offset=16, metric="euclidean"))
    elif kind == "pq_wide":      # the reference's own geometry: two sub-vectors of 64
        cfgs.append(sa.PQCacheConfig(heavy_size=64, pq_group_factor=2, pq_bits=6, kmeans_iter=4, init_offset=16, metric="euclidean"))
    fast = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    fast.return_attention_weights = False
    ref = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    m1, m2 = {}, {}
    kc, vc = k.to(cuda), v.to(cuda)
    calls = []
    orig = type(fast._plans).get

    for step in range(4):
        n = Lk + step
        qq = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=50 + step)[0].to(cuda)
        o1, w1 = fast.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=0)
        if kind.startswith("pq") and step == 0:
            # Both instances would take the general path here and cluster the keys; the Lloyd sums use floating-point
            # atomics, so two clusterings may differ in a last bit. The comparison is about the steps after it: the
            # second instance starts from a copy of the first one's codebook.
            m2 = copy.deepcopy(m1)
            continue
        o2, w2 = ref.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m2, layer_idx=0)
        assert w1 is None and w2 is not None
        if kind == "fixed":
            assert torch.equal(o1, o2), f"step {step}"
        elif kind == "hash":
            assert _same_output(o1, o2, B * Hq), f"step {step}"
        else:
            # selection and attention of these chains run as one kernel that deals a row's entries to its workgroups
            # in another order than the stand-alone attention: same columns, sums that may differ in a last bit
            plan = next(iter(fast._plans.values()))
            member = torch.zeros((B * Hq, n), dtype=torch.bool, device=cuda)
            member.scatter_(1, plan.cols[:, :int(plan.cnt[0])].long(), True)
            assert bool((plan.cnt == plan.cnt[0]).all()) and torch.equal(member.view(B, Hq, n), w2[:, :, 0] != 0), f"step {step}"
            assert rel_err(o1, o2) < 4e-3, f"step {step}"
    plan = next(iter(fast._plans.values()))
    assert plan.att.out is not None and plan.att.Lk == Lk + 3     # the last step went through the plan



def test_decode_plan_hashes_new_keys_in_blocks(cuda):
    """HashAttention decode through the plan: keys still inside the local window are hashed a block at a time
    (one bulk launch every `window` steps here), not one per step. Over enough steps for such keys to leave the
    window and compete, every output equals the masker-by-masker path's, which hashes one key per step, and the
    stored codes agree."""
    sa = _sa()
    dtype = torch.bfloat16
    B, Hq, Hkv, Lk, D = 2, 8, 2, 1500, 128
    steps, window = 40, 16
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk + steps, D, dtype, outliers=True, seed=11)
    cfgs = [sa.SinkMaskerConfig(sink_size=8), sa.LocalMaskerConfig(window_size=window),
            sa.HashAttentionTopKMaskerConfig(heavy_size=200, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                             hat_mlp_activation="silu", hat_weights=_hat(sa, Hq, D, dtype, hidden=128))]
    fast = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    fast.return_attention_weights = False
    ref = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    m1, m2 = {}, {}
    kc, vc = k.to(cuda), v.to(cuda)
    hashed = []
    for step in range(steps):
        n = Lk + step
        qq = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=150 + step)[0].to(cuda)
        o1, _ = fast.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=0)
        o2, _ = ref.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m2, layer_idx=0)
        assert _same_output(o1, o2, B * Hq), f"step {step}"
        c1, c2 = m1["key"][0], m2["key"][0]
        assert c2.n == n and n - window < c1.n <= n
        hashed.append(c1.n)
    assert len(set(hashed)) == 1 + (steps - 1) // window                 # the cold call, then one block per `window` steps
    assert torch.equal(c1.codes[:, :, : c1.n], c2.codes[:, :, : c1.n])


@pytest.mark.parametrize("n_sub", [16, 4])
def test_decode_plan_quantises_new_keys_in_blocks(cuda, n_sub):
    """PQCache decode through the plan: keys still inside the local window are quantised a block at a time (one
    launch every `window` steps here), and the scoring pass covers the quantised keys only. Over enough steps for
    such keys to leave the window and compete, every output equals the masker-by-masker path's, which quantises one
    key per step, and the stored codes agree."""
    sa = _sa()
    dtype = torch.bfloat16
    B, Hq, Hkv, Lk, D = 2, 8, 2, 1500, 128
    steps, window, off = 40, 16, 8
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk + steps, D, dtype, outliers=True, seed=13)
    cfgs = [sa.SinkMaskerConfig(sink_size=off), sa.LocalMaskerConfig(window_size=window),
            sa.PQCacheConfig(heavy_size=100, pq_group_factor=n_sub, pq_bits=6, kmeans_iter=3, init_offset=off, metric="euclidean")]
    fast = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    fast.return_attention_weights = False
    ref = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    m1 = {}
    kc, vc = k.to(cuda), v.to(cuda)
    fast.custom_attention(None, q[:, :, :1].to(cuda), kc[:, :, :Lk], vc[:, :, :Lk], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=0)
    m2 = copy.deepcopy(m1)          # both start from the same codebook
    quantised = []
    for step in range(1, steps):
        n = Lk + step
        qq = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=250 + step)[0].to(cuda)
        o1, _ = fast.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=0)
        o2, _ = ref.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m2, layer_idx=0)
        assert rel_err(o1, o2) < 4e-3, f"step {step}"      # same columns; the one-kernel form sums in another order
        b1, b2 = m1["pq_codebook"][0], m2["pq_codebook"][0]
        assert b2.n == n - off and n - off - window < b1.n <= n - off
        quantised.append(b1.n)
    assert len(set(quantised)) == 1 + (steps - 1) // window              # the cold call's count, then one block per `window` steps
    assert torch.equal(b1.codes[:, :, : b1.n], b2.codes[:, :, : b1.n])


def test_compact_code_stream_matches_two_plane_codes(cuda):
    """sah_hash_compact_codes: sign planes copied, every column with a zero component listed exactly once with
    both planes, counts right also beyond the list's capacity, ranges added in any order."""
    from sparse_attention_hub_amd import _native as N

    g = torch.Generator().manual_seed(5)
    n_rows, n, pitch, cap = 6, 5000, 5056, 64
    codes = torch.randint(-2**31, 2**31 - 1, (n_rows, pitch, 2), generator=g, dtype=torch.int64).to(torch.int32)
    zero = torch.rand((n_rows, pitch), generator=g) < torch.tensor([0.0, 0.001, 0.01, 0.01, 0.5, 1.0]).view(-1, 1)
    codes[..., 1] = torch.where(zero, codes[..., 1] & 0x7FFEFFFF, torch.full_like(codes[..., 1], -1))
    codes[..., 0] &= codes[..., 1]
    dc = codes.to(cuda)
    pos = torch.zeros((n_rows, pitch + 8192), dtype=torch.int32, device=cuda)
    exc = torch.zeros((n_rows, cap, 4), dtype=torch.int32, device=cuda)
    cnt = torch.zeros((n_rows,), dtype=torch.int32, device=cuda)
    for lo, hi in [(1000, 3000), (0, 1000), (3000, 3000), (3000, n)]:
        N.call("sah_hash_compact_codes", N.HashCompactArgs(dc.data_ptr(), pitch, n_rows, lo, hi, pos.data_ptr(), pos.shape[1],
                                                            exc.data_ptr(), cap, cnt.data_ptr(), 0xFFFFFFFF, N.stream_ptr(cuda)))
    assert torch.equal(pos[:, :n].cpu(), codes[:, :n, 0])
    assert not bool(pos[:, n:].any())
    want = [torch.nonzero(codes[r, :n, 1] != -1).flatten() for r in range(n_rows)]
    assert cnt.cpu().tolist() == [len(w) for w in want]
    e = exc.cpu()
    for r in range(n_rows):
        m = min(len(want[r]), cap)
        cols = e[r, :m, 0].long()
        assert len(set(cols.tolist())) == m and set(cols.tolist()) <= set(want[r].tolist())
        if len(want[r]) <= cap:
            assert sorted(cols.tolist()) == want[r].tolist()
        assert torch.equal(e[r, :m, 1], codes[r, cols, 1]) and torch.equal(e[r, :m, 2], codes[r, cols, 0])


@pytest.mark.parametrize("Lk,zero_key_bits,B", [(900, [5], 8), (2300, [0, 31], 8), (2300, [0, 31], 1), (1500, [], 8)])
def test_compact_codes_with_many_zero_components(cuda, Lk, zero_key_bits, B):
    """The decode kernel on the compact code stream when the exception list is long (a key bit that is zero for
    every key: all columns listed) or overflows (more than its 1024 entries: every column re-scored from the
    two-plane codes), with zero query components as well: outputs equal the masker-by-masker path's. B = 1: the
    selection kernel without the attention half."""
    sa = _sa()
    dtype = torch.bfloat16
    Hq, Hkv, D = 32, 8, 128
    wts = _hat(sa, Hq, D, dtype, hidden=128)
    for e in zero_key_bits:
        wts[0]["key_matrix"][-1][..., e] = 0
        wts[0]["key_bias"][-1][..., e] = 0
    wts[0]["query_matrix"][-1][..., 9] = 0
    wts[0]["query_bias"][-1][..., 9] = 0
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk + 3, D, dtype, outliers=True, seed=31)
    cfgs = [sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=64),
            sa.HashAttentionTopKMaskerConfig(heavy_size=200, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                             hat_mlp_activation="silu", hat_weights=wts)]
    fast = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    fast.return_attention_weights = False
    ref = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    m1, m2 = {}, {}
    kc, vc = k.to(cuda), v.to(cuda)
    for step in range(3):
        n = Lk + step
        qq = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=350 + step)[0].to(cuda)
        o1, _ = fast.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=0)
        o2, _ = ref.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m2, layer_idx=0)
        assert _same_output(o1, o2, B * Hq), f"step {step}"
    cache = m1["key"][0]
    assert cache.n_compact == Lk and cache.exc.shape[2] == 1024
    listed = cache.exc_cnt.cpu()
    if zero_key_bits:
        assert bool((listed == Lk).all())            # every key has a zero component: listed, or overflowed
    else:
        assert 0 < int(listed.max()) < 200           # bf16 outputs that round to exactly zero: a few per row


def test_hash_decode_plan_state_transitions(cuda):
    """The HashAttention decode plan keeps state between steps (keys hashed so far, the compact copy of the codes).
    Every transition that touches it: plan steps with unhashed keys pending, then a call that takes the
    masker-by-masker path (it must hash what is missing), back to the plan (the compact copy catches up), a cache
    that is reallocated (the compact copy is rebuilt), two layers interleaved. Outputs always equal those of a
    second instance that never uses the plan."""
    sa = _sa()
    dtype = torch.bfloat16
    B, Hq, Hkv, Lk, D = 8, 32, 8, 1200, 128
    steps = 30
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk + steps, D, dtype, outliers=True, seed=41)
    wts = {0: _hat(sa, Hq, D, dtype, hidden=128, seed=1)[0], 1: _hat(sa, Hq, D, dtype, hidden=128, seed=2)[0]}
    cfgs = [sa.SinkMaskerConfig(sink_size=8), sa.LocalMaskerConfig(window_size=8),
            sa.HashAttentionTopKMaskerConfig(heavy_size=150, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                             hat_mlp_activation="silu", hat_weights=wts)]
    fast = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    ref = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    m1, m2 = {}, {}
    kc, vc = k.to(cuda), v.to(cuda)
    seen_lag = regrown = False
    for step in range(steps):
        n = Lk + step
        general = step in (5, 6, 17)                     # these steps ask for the weights: masker-by-masker path
        fast.return_attention_weights = general
        for layer in (0, 1):
            qq = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=450 + 2 * step + layer)[0].to(cuda)
            o1, w1 = fast.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=layer)
            o2, w2 = ref.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m2, layer_idx=layer)
            assert _same_output(o1, o2, B * Hq), f"step {step} layer {layer}"
            assert (w1 is not None) == general
            if general:
                assert torch.equal(w1, w2)
                assert m1["key"][layer].n == n           # the general path hashed the pending keys
        cache = m1["key"][0]
        seen_lag |= cache.n < n
        if step == 11:                                   # force a reallocation of the code cache
            cache.reserve(cache.capacity + 1)
            assert cache.pos is None and cache.n_compact == 0
            regrown = True
        if step > 12 and not general:
            assert cache.pos is not None and cache.n_compact == cache.n
    assert seen_lag and regrown
    for layer in (0, 1):
        c1, c2 = m1["key"][layer], m2["key"][layer]
        assert torch.equal(c1.codes[:, :, : c1.n], c2.codes[:, :, : c1.n])
        assert torch.equal(c1.pos[:, :, : c1.n_compact], c1.codes[:, :, : c1.n_compact, 0])
        zeros = (c1.codes[:, :, : c1.n_compact, 1] != -1).sum(-1)
        assert torch.equal(zeros.to(torch.int32), c1.exc_cnt)


@pytest.mark.parametrize("case", [
    # bits, n, k, active, columns whose code equals the query's (score 32: the highest threshold bracket)
    (32, 5000, 5, 40, 9),          # threshold = the top score itself, ties cut among the 9
    (32, 5000, 9, 40, 9),
    (32, 5000, 300, 40, 9),        # usual case: threshold a few steps above the mean
    (32, 3000, 2500, 100, 0),      # most of the row: threshold below the mean (second probe set)
    (4, 4000, 3000, 10, 0),        # 4-bit signatures: scores + 33 in [29, 37], heavy ties
    (32, 700, 690, 20, 0),         # more wanted than exist: every inactive column
    (32, 40000, 2048, 640, 3),     # two mask groups per wave
])
def test_hamming_topk_threshold_brackets(cuda, case):
    """sah_hamming_topk against a stable descending sort of the reference's signature score, on code sets built
    to put the threshold in each of the ranges the kernel resolves differently (top score, usual range, below the
    mean, nothing left), ties to the lowest column."""
    from sparse_attention_hub_amd import _native as N
    from sparse_attention_hub_amd.sparse_attention.utils.native_rows import NativeRows

    bits, n, k, n_active, n_same = case
    R = 3
    g = torch.Generator().manual_seed(bits * 1000 + k)
    mask = (1 << bits) - 1
    pitch = n + (n % 2)
    kc = torch.randint(0, 2**31 - 1, (R, pitch, 2), generator=g, dtype=torch.int64) * 2 + torch.randint(0, 2, (R, pitch, 2), generator=g)
    kc &= mask
    qc = (torch.randint(0, 2**31 - 1, (R, 2), generator=g, dtype=torch.int64) * 2 + 1) & mask
    kc[..., 1] = mask
    qc[..., 1] = mask
    for r in range(R):
        same = torch.randperm(n, generator=g)[:n_same]
        kc[r, same, 0] = qc[r, 0]
    rows = NativeRows(R, n, n_active + k, cuda)
    rows.zero_if_fresh()
    act = torch.zeros(R, n, dtype=torch.bool)
    cols = torch.zeros((R, n_active), dtype=torch.int32)
    for r in range(R):
        idx = torch.randperm(n, generator=g)[:n_active]
        act[r, idx] = True
        cols[r] = idx.to(torch.int32)
    rows.cols[:, :n_active] = cols.to(cuda)
    rows.cnt.fill_(n_active)
    words = torch.zeros((R, rows.bitmap.shape[1] * 32), dtype=torch.bool)
    words[:, :n] = act
    packed = (words.view(R, -1, 32).to(torch.int64) << torch.arange(32, dtype=torch.int64)).sum(-1)
    rows.bitmap.copy_(torch.where(packed >= 2**31, packed - 2**32, packed).to(torch.int32).to(cuda))
    rows.max_cnt = n_active
    rows.fresh = False
    to_i32 = lambda t: torch.where(t >= 2**31, t - 2**32, t).to(torch.int32)
    dk, dq = to_i32(kc).contiguous().to(cuda), to_i32(qc).contiguous().to(cuda)
    N.call("sah_hamming_topk", N.HammingTopkArgs(rows.as_struct(), dk.data_ptr(), pitch, dq.data_ptr(), 1, k, N.stream_ptr(cuda)))
    sc = O.signature_scores_from_codes(qc.view(R, 1, 2), kc[:, :n]).view(R, n).float()
    sc[act] = float("-inf")
    want = O.stable_topk(sc, min(k, n))
    got_cnt = rows.cnt.cpu()
    got_cols = rows.cols.cpu()
    for r in range(R):
        exp = sorted(want[r].tolist()[: min(k, n - n_active)])     # active columns score -inf and sort last
        got = sorted(got_cols[r, n_active: int(got_cnt[r])].tolist())
        assert int(got_cnt[r]) == n_active + len(exp) and got == exp, f"row {r}"


def test_pq_clustering_is_reproducible(cuda):
    """Two clusterings of the same keys give the same centroids and codes, bit for bit: the Lloyd sums are
    order-independent (64-bit fixed point), whatever order workgroups and waves add in."""
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.utils.pq_utils import kmeans_keys_batched

    B, Hkv, n, D, n_sub, n_cent = 2, 4, 20000, 128, 16, 256
    k = make_qkv(B, Hkv, Hkv, 1, n, D, torch.bfloat16, outliers=True, seed=77)[1].to(cuda)
    runs = []
    for _ in range(3):
        codes = torch.zeros((B, Hkv, n, n_sub), dtype=torch.uint8, device=cuda)
        centres, _ = kmeans_keys_batched(k, 0, n_sub, n_cent, 4, codes, n, seed=3)
        runs.append((centres.clone(), codes.clone()))
    for c, z in runs[1:]:
        assert torch.equal(c, runs[0][0]) and torch.equal(z, runs[0][1])


def test_oracle_topk_full_size_properties(cuda):
    """Config 2 at its full shape (B = 4, 32 query / 8 KV heads, 32768 keys, top 5 % = 1638, bf16), checked
    through properties that need no CPU restatement of 128 x 32768 scores: every row holds sink + local +
    k distinct columns, the sink and local columns among them, and the chosen columns dominate the rest
    in the kernel's own order-preserving score keys (ties to the lowest column)."""
    sa = _sa()
    dtype = torch.bfloat16
    B, Hq, Hkv, Lk, D = 4, 32, 8, 32768, 128
    sink, window, k_eff = 128, 512, int(0.05 * 32768)
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, outliers=True, seed=3)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(
        masker_configs=[sa.SinkMaskerConfig(sink_size=sink), sa.LocalMaskerConfig(window_size=window), sa.OracleTopKConfig(heavy_size=0.05)]))
    ra.return_attention_weights = False
    out, _ = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data={}, layer_idx=0)
    plan = next(iter(ra._plans.values()))
    n_rows = B * Hq
    cnt = plan.cnt.cpu()
    assert bool((cnt == sink + window + k_eff).all())
    cols = plan.cols[:, : sink + window + k_eff].long()
    srt = torch.sort(cols, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all()) and int(cols.min()) == 0 and int(cols.max()) == Lk - 1
    member = torch.zeros((n_rows, Lk), dtype=torch.bool, device=cuda)
    member.scatter_(1, cols, True)
    assert bool(member[:, :sink].all()) and bool(member[:, Lk - window:].all())
    keys = (plan.keybuf[:, :Lk].to(torch.int32) & 0xFFFF)             # sortable keys: larger = better
    cand = keys.clone()
    cand[:, :sink] = -1
    cand[:, Lk - window:] = -1
    chosen = member.clone()
    chosen[:, :sink] = False
    chosen[:, Lk - window:] = False
    assert bool((chosen.sum(1) == k_eff).all())
    lowest_in = torch.where(chosen, cand, torch.full_like(cand, 1 << 20)).min(1).values
    highest_out = torch.where(chosen, torch.full_like(cand, -1), cand).max(1).values
    assert bool((lowest_in >= highest_out).all())
    # ties at the threshold: every column left out with the threshold key lies behind every chosen one with that key
    T = lowest_in.unsqueeze(1)
    idx = torch.arange(Lk, device=cuda).unsqueeze(0).expand(n_rows, -1)
    last_in = torch.where(chosen & (cand == T), idx, torch.full_like(idx, -1)).max(1).values
    first_out = torch.where(~chosen & (cand == T), idx, torch.full_like(idx, Lk)).min(1).values
    assert bool((last_in < first_out).all())
    assert bool(torch.isfinite(out.float()).all())


def _set_hash_block(monkeypatch, block, compact=None):
    """New keys per bulk hashing launch of the decode plan (1 = the newest key is hashed inside every step's
    kernel) and whether the kernel scans the compact code stream (default: whenever keys are hashed in blocks)."""
    import importlib

    plan_mod = importlib.import_module("sparse_attention_hub_amd.sparse_attention.research_attention.decode_plan")
    monkeypatch.setattr(plan_mod, "_HASH_BLOCK", block)
    monkeypatch.setattr(plan_mod, "_COMPACT_CODES", block != 1 if compact is None else compact)


@pytest.mark.parametrize("block,compact", [(1, False), (64, True), (64, False), (1, True)])
@pytest.mark.parametrize("dtype,Lk", [(torch.bfloat16, 32768), (torch.float16, 5000), (torch.float32, 3001), (torch.bfloat16, 70001)])
def test_fused_hash_decode_kernel_matches_separate_launches(cuda, monkeypatch, dtype, Lk, block, compact):
    """Sink + Local + HashAttention decode steps through the single fused kernel (sink/local rows, both signature
    MLPs, signature top-k) against the masker-by-masker path: same outputs, same signature cache, bit for bit,
    at the headline shape (32 query heads, 8 KV heads, 32768 keys, top-2048) and at ragged sizes."""
    from sparse_attention_hub_amd import _native as N

    sa = _sa()
    _set_hash_block(monkeypatch, block, compact)
    # 256 rows at the ragged size: one workgroup per row; 64 and 32 rows at the longer ones: four and eight per row
    B, Hq, Hkv, D = (8 if Lk <= 8192 else 2 if Lk <= 32768 else 1), 32, 8, 128   # 70001 keys: 18 chunks per wave
    heavy = 2048 if Lk > 8192 else 300
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk + 3, D, dtype, seed=3)
    cfgs = [sa.SinkMaskerConfig(sink_size=128), sa.LocalMaskerConfig(window_size=512),
            sa.HashAttentionTopKMaskerConfig(heavy_size=heavy, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                             hat_mlp_activation="silu", hat_weights=_hat(sa, Hq, D, dtype, hidden=128))]
    fast = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    fast.return_attention_weights = False
    ref = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    m1, m2 = {}, {}
    kc, vc = k.to(cuda), v.to(cuda)
    for step in range(3):
        n = Lk + step
        qq = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=70 + step)[0].to(cuda)
        if step == 2:
            N.timing_enable(True)
        o1, _ = fast.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=0)
        if step == 2:
            torch.cuda.synchronize()
            names = set(N.timing_collect())
            N.timing_enable(False)
            if block == 1 and compact:   # the new key is hashed and added to the compact stream by launches of their own
                names -= {"k_hash_compact", "k_hash_sig_small_mfma", "k_hash_sig_gemv"}
            # the whole step, attention included, is one kernel: one workgroup per row, or - with fewer rows than
            # compute units - several per row whose partial results the last one to finish merges
            assert names == {"k_hash_decode_attn"}, names
        o2, _ = ref.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m2, layer_idx=0)
        assert _same_output(o1, o2, B * Hq), f"step {step}"
        hashed = m1["key"][0].n                                       # block > 1: the newest keys are not hashed yet
        assert hashed == (n if block == 1 else Lk)
        assert torch.equal(m1["key"][0].codes[:, :, :hashed], m2["key"][0].codes[:, :, :hashed]), f"cache, step {step}"
    # the rows the fused kernel built: sink + local + top-k entries, all distinct
    plan = next(iter(fast._plans.values()))
    cnt = plan.cnt.cpu()
    assert bool((cnt == 128 + 512 + heavy).all())
    cols = plan.cols[:, : 128 + 512 + heavy].long()
    srt = torch.sort(cols, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all()) and int(cols.min()) == 0 and int(cols.max()) == Lk + 2 - 1


@pytest.mark.parametrize("case", [
    # n_keys, n_cand, col_offset, k, distinct key values (0 = all 65536), active per row, excluded key
    (700, 700, 0, 50, 0, 30, 0x0080),
    (700, 690, 10, 50, 20, 30, 0),          # heavy ties, candidate range not aligned to anything
    (1300, 1283, 17, 200, 5, 100, 3),        # the excluded key lies inside the tie range: active columns take rank
    (5000, 4872, 128, 600, 300, 640, 0),
    (100, 100, 0, 100, 9, 40, 4),            # k = all candidates
    (37, 30, 7, 3, 9, 0, 0),
    (40000, 39990, 10, 2048, 3000, 640, 0x0080),   # 5 chunks per wave
    (70016, 70000, 16, 3000, 40, 700, 7),          # 9 chunks per wave, ties everywhere
    (140000, 139999, 1, 5000, 0, 300, 0x0080),     # too long for registers: keys re-read per pass
    # distinct key values = -(1 + j): float-like keys, the k-th largest lies j high-byte bins below the row's largest
    # (the threshold search looks at the largest key's bin and the next, then at two more, then builds histograms)
    (6000, 6000, 0, 300, -1, 40, 0x0080),
    (6000, 5990, 10, 300, -2, 40, 0x0080),
    (6000, 6000, 0, 300, -3, 40, 0),
    (20000, 19999, 1, 1000, -4, 640, 0x0080),
    (6000, 6000, 0, 300, -6, 40, 0x0080),
    (33000, 33000, 0, 300, -4, 40, 0x0080),        # the same with 5 chunks per wave
])
def test_select_topk_16bit_keys_against_stable_sort(cuda, case):
    """sah_select_topk on 16-bit keys, straight through the C ABI: the k best candidates in the order
    (key descending, column ascending), columns already active ranking with the excluded key and never
    emitted again; rows, counts and bitmap against a stable sort on the host."""
    import numpy as np

    from sparse_attention_hub_amd import _native as N

    n_keys, n_cand, off, k, n_vals, n_active, ek = case
    n_rows = 3 if n_keys < 20000 else 2
    rng = np.random.default_rng(n_keys + k)
    pitch = (n_cand + 7) // 8 * 8
    if n_vals < 0:
        j, top = -n_vals - 1, 0xC9
        # fewer than k keys in the j bins from the largest key's down, most of the row in the bin below them (low bytes
        # from a small set, so the threshold is tied) and the rest spread over the bins further down
        hi = rng.integers(top - j - 40, top - j + 1, size=(n_rows, pitch))
        hi[rng.random((n_rows, pitch)) < 0.5] = top - j
        few = rng.random((n_rows, pitch)) < (0.5 * k / n_cand)
        hi[few] = rng.integers(top - j + 1, top + 1, size=int(few.sum())) if j else top
        hi[:, 5] = top
        keys = ((hi << 8) | rng.integers(0, 256, size=(n_rows, pitch)) // 8 * 8).astype(np.uint16)
    elif n_vals:
        keys = rng.integers(1, n_vals + 1, size=(n_rows, pitch)).astype(np.uint16)
    else:
        keys = rng.integers(0, 65536, size=(n_rows, pitch)).astype(np.uint16)
    n_words = (n_keys + 31) // 32
    cap = min(n_keys, n_active + k)
    cols = np.full((n_rows, cap), -1, np.int32)
    bm = np.zeros((n_rows, n_words), np.uint32)
    active = []
    for r in range(n_rows):
        a = rng.choice(n_keys, size=n_active, replace=False) if n_active else np.zeros(0, np.int64)
        active.append(set(a.tolist()))
        cols[r, :n_active] = a
        for c in a:
            bm[r, c >> 5] |= np.uint32(1 << (c & 31))
    tk = torch.from_numpy(keys.view(np.int16)).to(cuda)
    tc = torch.from_numpy(cols).to(cuda)
    tn = torch.full((n_rows,), n_active, dtype=torch.int32, device=cuda)
    tb = torch.from_numpy(bm.view(np.int32)).to(cuda)
    rows = N.Rows(tc.data_ptr(), tn.data_ptr(), None, tb.data_ptr(), n_rows, cap, n_keys, n_words)
    N.call("sah_select_topk", N.SelectTopkArgs(rows, tk.data_ptr(), pitch, 16, n_cand, off, k, ek, 0, 0, 0, N.stream_ptr(cuda)))
    torch.cuda.synchronize()
    got_cols, got_cnt, got_bm = tc.cpu().numpy(), tn.cpu().numpy(), tb.cpu().numpy().view(np.uint32)
    for r in range(n_rows):
        eff = keys[r, :n_cand].astype(np.int64)
        excl = np.zeros(n_cand, bool)
        for c in active[r]:
            if off <= c < off + n_cand:
                excl[c - off] = True
        eff[excl] = ek
        order = np.argsort(-eff, kind="stable")[: min(k, n_cand)]
        want = set((order[~excl[order]] + off).tolist())
        new = got_cols[r, n_active:got_cnt[r]].tolist()
        assert got_cnt[r] == n_active + len(want) and set(new) == want and len(new) == len(want), f"row {r}"
        assert set(got_cols[r, :n_active].tolist()) == active[r]
        exp = bm[r].copy()
        for c in want:
            exp[c >> 5] |= np.uint32(1 << (c & 31))
        assert np.array_equal(got_bm[r], exp), f"bitmap, row {r}"


@pytest.mark.parametrize("key_bits", [16, 32])
def test_select_topk_on_fresh_rows_equals_sink_local_then_select(cuda, key_bits):
    """sah_select_topk with fresh != 0 writes the sink + local rows itself (inside the selection kernel for
    16-bit keys, by a launch of its own otherwise): same rows, counts and bitmap as the two calls."""
    from sparse_attention_hub_amd import _native as N
    from sparse_attention_hub_amd.sparse_attention.utils.native_rows import NativeRows

    n_rows, n_keys, sink, window, k = 6, 3001, 37, 211, 150
    g = torch.Generator().manual_seed(5)
    hi = 1 << (key_bits - 4)
    keys = torch.randint(0, hi, (n_rows, 3008), generator=g, dtype=torch.int64)
    kdev = keys.to(torch.int16 if key_bits == 16 else torch.int32).to(cuda)
    results = []
    for fused in (True, False):
        rows = NativeRows(n_rows, n_keys, sink + window + k, cuda)
        if not fused:
            N.call("sah_sink_local_indices", N.SinkLocalArgs(rows.as_struct(), 1, sink, window, 1, 0, N.stream_ptr(cuda)))
        args = N.SelectTopkArgs(rows.as_struct(), kdev.data_ptr(), kdev.stride(0), key_bits, n_keys, 0, k, 0,
                                1 if fused else 0, sink if fused else 0, window if fused else 0, N.stream_ptr(cuda))
        N.call("sah_select_topk", args)
        torch.cuda.synchronize()
        results.append((rows.cnt.cpu(), torch.sort(rows.cols.cpu(), dim=1).values, rows.bitmap.cpu()))
    (c1, s1, b1), (c2, s2, b2) = results
    assert bool((c1 == sink + window + k).all()) and torch.equal(c1, c2)
    assert torch.equal(s1, s2) and torch.equal(b1, b2)
    # and against a plain restatement: best k of the columns outside sink and window, lowest column on ties
    kk = keys[:, :n_keys].clone()
    kk[:, :sink] = -1
    kk[:, n_keys - window:] = -1
    want = torch.argsort(kk, dim=1, descending=True, stable=True)[:, :k]
    got = torch.stack([row[(row >= sink) & (row < n_keys - window)] for row in s1])
    assert torch.equal(got, torch.sort(want, dim=1).values.to(got.dtype))


def test_density_and_output_error_metrics(cuda, tmp_path):
    """research_attention_density and research_attention_output_error (reference research_attention/base.py:
    121-126, 150-168) through the kernels: density = entries / (rows * keys) exactly, error = relative
    distance between the sparse output and dense attention, against the oracle's two outputs."""
    import json

    from sparse_attention_hub_amd.metric_logging import MicroMetricLogger

    sa = _sa()
    B, Hq, Hkv, Lk, D = 2, 8, 2, 900, 64
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, torch.float32, seed=21)
    cfgs = [sa.SinkMaskerConfig(sink_size=8), sa.LocalMaskerConfig(window_size=32), sa.OracleTopKConfig(heavy_size=60)]
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    ra.return_attention_weights = False   # the metrics must also work when the fast decode plan would apply
    lg = MicroMetricLogger()
    saved = (lg.log_path, set(lg.enabled_metrics), lg.max_records, lg.sampling_factor)
    try:
        lg.configure_logging(str(tmp_path), enabled_metrics=["research_attention_density", "research_attention_output_error"])
        out, _ = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5, 0.0, sparse_meta_data={}, layer_idx=3)
        lg.flush()
    finally:
        lg.log_path, lg.enabled_metrics, lg.max_records, lg.sampling_factor = saved
    recs = [json.loads(line) for line in (tmp_path / "micro_metrics.jsonl").read_text().splitlines()]
    assert [r["metric"] for r in recs] == ["research_attention_density", "research_attention_output_error"]
    assert all(r["metadata"] == {"layer_idx": 3} for r in recs)
    assert all(r["location"].endswith("ResearchAttention.custom_attention") for r in recs)
    assert recs[0]["value"] == pytest.approx((8 + 32 + 60) / Lk, rel=1e-6)
    o_sparse, _, _ = O.research_attention([("sink", 8), ("local", 32), ("oracle_topk", 60)], q, k, v, None, D ** -0.5, None)
    o_dense, _, _ = O.research_attention([], q, k, v, None, D ** -0.5, None)
    want = (torch.norm(o_dense - o_sparse) / torch.norm(o_dense)).item()
    assert recs[1]["value"] == pytest.approx(want, rel=1e-3)
    assert torch.allclose(out.cpu(), o_sparse, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("block", [1, 64])
def test_single_kernel_decode_step_head_dim_64(cuda, monkeypatch, block):
    """The one-kernel decode step (selection + attention) at head_dim 64 with 64-wide signature layers,
    256 mask rows, a context that is not a multiple of anything: outputs and cache equal to the
    masker-by-masker path, and against the oracle given the kernel's signatures."""
    from sparse_attention_hub_amd import _native as N

    sa = _sa()
    _set_hash_block(monkeypatch, block)
    dtype = torch.bfloat16
    B, Hq, Hkv, D, Lk = 8, 32, 8, 64, 1237
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk + 2, D, dtype, seed=13)
    cfgs = [sa.SinkMaskerConfig(sink_size=20), sa.LocalMaskerConfig(window_size=70),
            sa.HashAttentionTopKMaskerConfig(heavy_size=150, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=64,
                                             hat_mlp_activation="silu", hat_weights=_hat(sa, Hq, D, dtype, hidden=64))]
    fast = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    fast.return_attention_weights = False
    ref = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    m1, m2 = {}, {}
    kc, vc = k.to(cuda), v.to(cuda)
    for step in range(2):
        n = Lk + step
        qq = make_qkv(B, Hq, Hkv, 1, 1, D, dtype, seed=40 + step)[0].to(cuda)
        if step == 1:
            N.timing_enable(True)
        o1, _ = fast.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m1, layer_idx=0)
        if step == 1:
            torch.cuda.synchronize()
            names = set(N.timing_collect())
            N.timing_enable(False)
            assert names - {"k_hash_compact"} == {"k_hash_decode_attn"}, names   # first plan step: the compact stream is built
        o2, w2 = ref.custom_attention(None, qq, kc[:, :, :n], vc[:, :, :n], None, D ** -0.5, 0.0, sparse_meta_data=m2, layer_idx=0)
        assert torch.equal(o1, o2), f"step {step}"
        hashed = m1["key"][0].n
        assert hashed == (n if block == 1 else Lk)
        assert torch.equal(m1["key"][0].codes[:, :, :hashed], m2["key"][0].codes[:, :, :hashed]), f"cache, step {step}"
        assert bool(((w2 != 0).sum(-1) == 20 + 70 + 150).all())


# ------------------------------------------------------------------------ adaptive sampling
def _adaptive_case(cuda, pre_cfgs, pre_specs, rate, eps, delta, io, lo, B, Hq, Hkv, Lq, Lk, D, dtype, amask=None,
                   seed=1234, outliers=False):
    sa = _sa()
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, dtype, seed=5, outliers=outliers)
    acfg = sa.AdaptiveSamplingMaskerConfig(base_rate_sampling=rate, epsilon=eps, delta=delta, init_offset=io,
                                           local_offset=lo)
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=pre_cfgs + [acfg]))
    masker = ra.maskers[-1]
    masker.seed = seed
    scaling = D ** -0.5
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None if amask is None else amask.to(cuda),
                                 scaling, 0.0, sparse_meta_data={}, layer_idx=0)
    torch.cuda.synchronize()
    specs = pre_specs + [("adaptive", rate, eps, delta, io, lo, seed, 0)]
    # 1) the budget: float arithmetic in the tensor dtype, compared with the oracle's
    st = {}
    O.research_attention(specs, q, k, v, amask, scaling, None, st)
    b_oracle = st["budget_oracle"].reshape(-1)
    b_kernel = masker.last_budget.cpu().long()
    return q, k, v, out, w, specs, scaling, b_kernel, b_oracle


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chain", ["alone", "sink_local", "oracle", "amask", "lq2"])
def test_adaptive_sampling_chain(cuda, dtype, chain):
    """Budgets agree with the oracle (they are floats truncated to integers: a last-place difference in a sum
    may move one by a unit of its precision); given the kernel's budgets, the sampled index sets are bit-exact
    and outputs are within tolerance."""
    sa = _sa()
    pre_cfgs, pre_specs, amask = [], [], None
    B, Hq, Hkv, Lq, Lk, D = 2, 4, 2, 1, 1500, 32
    io, lo = 0, 0
    if chain != "alone":
        pre_cfgs = [sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=32)]
        pre_specs = [("sink", 16), ("local", 32)]
        io, lo = 16, 32
    if chain == "oracle":
        pre_cfgs.append(sa.OracleTopKConfig(heavy_size=0.02))
        pre_specs.append(("oracle_topk", 0.02))
    if chain == "amask":
        amask = torch.zeros(B, 1, Lq, Lk)
        amask[..., 900:1000] = -1e4
        amask = amask.to(dtype)
    if chain == "lq2":
        Lq, io, lo = 2, 0.01, 0.02
    q, k, v, out, w, specs, scaling, b_kernel, b_oracle = _adaptive_case(
        cuda, pre_cfgs, pre_specs, 0.02, 0.1, 0.1, io, lo, B, Hq, Hkv, Lq, Lk, D, dtype, amask)
    n = O.adaptive_sampling_range(Lk, io, lo)[2]
    nb = O.adaptive_base_count(0.02, n)
    assert int(b_kernel.min()) >= nb and int(b_kernel.max()) <= n
    assert int(b_kernel.max()) > nb  # the case exercises the formula, not only its lower clamp
    unit = (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -20)
    close = (b_kernel - b_oracle).abs().double() <= 1 + 2 * unit * b_oracle.double()
    assert bool(close.all()), (b_kernel.tolist(), b_oracle.tolist())
    assert float((b_kernel == b_oracle).double().mean()) >= 0.75
    # 2) index sets and outputs for the kernel's own budgets
    oo, ow, om = O.research_attention(specs, q, k, v, amask, scaling, None, {"budget": b_kernel})
    assert torch.equal(w.cpu() != 0, ow != 0)
    assert rel_err(out, oo) < TOL[dtype]
    assert (w.float().cpu() - ow.float()).abs().max().item() < (1e-6 if dtype == torch.float32 else 1e-2)


def test_adaptive_sampling_mask_weights_and_reproducibility(cuda):
    """The dense form of the final mask equals the oracle's (weights included), torch.manual_seed reseeds the
    sampler, and consecutive calls draw fresh samples."""
    sa = _sa()
    B, Hq, Hkv, Lq, Lk, D = 1, 4, 2, 1, 800, 16
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, torch.float32, seed=9)
    cfg = sa.AdaptiveSamplingMaskerConfig(base_rate_sampling=0.05, epsilon=0.2, delta=0.2, init_offset=8, local_offset=8)
    masks = []
    for rep in range(3):
        if rep < 2:
            torch.manual_seed(77)
        m = sa.AdaptiveSamplingMasker(cfg)
        prev = sa.Mask.create_empty_mask((B, Hq, Lq, Lk), torch.float32, cuda)
        prev = sa.SinkMasker(sa.SinkMaskerConfig(sink_size=8)).add_mask(k.to(cuda), q.to(cuda), v.to(cuda), None, 0.25, 0.0, {}, prev)
        first = m.add_mask(k.to(cuda), q.to(cuda), v.to(cuda), None, 0.25, 0.0, {}, prev).get_dense_mask().cpu()
        masks.append(first)
        if rep == 0:
            om, budget, prob = O.adaptive_sampling(O.sink(O.OMask.empty((B, Hq, Lq, Lk), torch.float32), 8), q, k, None,
                                                   0.25, 0.05, 0.2, 0.2, 8, 8, seed=77, offset=0,
                                                   budget_override=m.last_budget.cpu().long())
            assert torch.equal(first, om.to_dense())
            again = m.add_mask(k.to(cuda), q.to(cuda), v.to(cuda), None, 0.25, 0.0, {},
                               sa.Mask.create_empty_mask((B, Hq, Lq, Lk), torch.float32, cuda)).get_dense_mask().cpu()
            assert not torch.equal(again != 0, first != 0)
    assert torch.equal(masks[0], masks[1])
    assert not torch.equal(masks[0], masks[2]) or torch.initial_seed() == 77


def test_adaptive_sampling_denominator_guarantee_at_scale(cuda):
    """Size-independent property on a long context: the importance-weighted sum over the sampled mask estimates the
    full softmax denominator within epsilon for at least (1 - delta) of the rows (with slack for the normal
    approximation), and the rows' entries are distinct and inside the key range."""
    sa = _sa()
    B, Hq, Hkv, Lq, Lk, D = 2, 32, 8, 1, 32768, 128
    eps, delta = 0.1, 0.1
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, torch.bfloat16, seed=21, outliers=False, device=cuda)
    q = q * 0.5
    cfgs = [sa.SinkMaskerConfig(sink_size=128), sa.LocalMaskerConfig(window_size=512),
            sa.OracleTopKConfig(heavy_size=0.02),
            sa.AdaptiveSamplingMaskerConfig(base_rate_sampling=0.01, epsilon=eps, delta=delta, init_offset=128,
                                            local_offset=512)]
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
    n = Lk - 128 - 512
    fixed = 128 + 512 + int(0.02 * Lk)
    assert int(budget.min()) >= int(0.01 * n) and int(budget.max()) <= n
    assert bool((cnt <= fixed + budget).all()) and bool((cnt > fixed).all())
    # weighted estimate of the denominator against the exact one, in fp64 on the device
    kk = k.double().repeat_interleave(Hq // Hkv, dim=1)
    z = torch.matmul(q.double(), kk.transpose(-1, -2)) * scaling
    e = torch.exp(z - z.amax(dim=-1, keepdim=True)).reshape(B * Hq, Lk)
    true_den = e.sum(dim=-1)
    cols = rows.cols.long()
    pos = torch.arange(rows.cap, device=cuda).unsqueeze(0)
    valid = pos < rows.cnt.long().unsqueeze(1)
    wts = rows.w.double()
    est = (torch.where(valid, torch.gather(e, 1, cols.clamp(0, Lk - 1)) / wts.clamp_min(1e-9), torch.zeros_like(wts))).sum(dim=-1)
    rel = ((est - true_den).abs() / true_den).cpu()
    assert float((rel <= eps).double().mean()) >= 1.0 - delta - 0.08, float((rel <= eps).double().mean())
    # entries are distinct and in range
    big = torch.where(valid, cols, torch.full_like(cols, Lk + 1) + pos)
    srt = torch.sort(big, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all())
    assert bool(((cols >= 0) & (cols < Lk) | ~valid).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", ["small", "beyond_the_register_copies"])
def test_adaptive_budget_row_maximum_from_the_rows_entries(cuda, dtype, shape, monkeypatch):
    """After an exact top-k over the score keys the row maximum is among the row's entries: the budget kernel then
    skips its pass over all keys (`max_in_rows`). Budgets, probabilities and statistics must not change by a bit;
    the larger shape has more than 4096 entries per row and more than 4096 base draws (the parts of both that a
    thread does not keep in registers)."""
    sa = _sa()
    if shape == "small":
        B, Hq, Hkv, Lk, D, heavy, rate = 2, 4, 2, 3000, 32, 0.05, 0.05
    else:
        B, Hq, Hkv, Lk, D, heavy, rate = 1, 2, 1, 12000, 32, 5000, 0.75
    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=23)
    scaling = D ** -0.5

    def run():
        cfgs = [sa.SinkMaskerConfig(sink_size=8), sa.LocalMaskerConfig(window_size=16), sa.OracleTopKConfig(heavy_size=heavy),
                sa.AdaptiveSamplingMaskerConfig(base_rate_sampling=rate, epsilon=0.25, delta=0.25, init_offset=8, local_offset=16)]
        ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
        m = ra.maskers[-1]
        m.seed, m.keep_stats = 5, True
        out, _ = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, scaling, 0.0, sparse_meta_data={}, layer_idx=0)
        return out.cpu(), m.last_budget.cpu(), m.last_probability.cpu(), m.last_stats.cpu(), m.last_rows.cnt.cpu()

    from sparse_attention_hub_amd import _native as N

    seen = []
    orig_call = N.call

    def spy(name, args):
        if name == "sah_adaptive_budget":
            seen.append(int(args.max_in_rows))
        return orig_call(name, args)

    monkeypatch.setattr(N, "call", spy)
    with_flag = run()
    orig_add = sa.OracleTopK.add_mask

    def without_promise(self, *a, **kw):
        mask = orig_add(self, *a, **kw)
        kw["_call_scratch"].pop("qk_top_in_rows", None)
        return mask

    monkeypatch.setattr(sa.OracleTopK, "add_mask", without_promise)
    without_flag = run()
    assert seen == [1, 0]
    for a, b in zip(with_flag, without_flag):
        assert torch.equal(a, b)
    if shape != "small":
        assert int(with_flag[4].min()) > 4096 + 24


def test_adaptive_sampling_abi_rejects_bad_arguments(cuda):
    from sparse_attention_hub_amd import _native as N
    from sparse_attention_hub_amd.sparse_attention.utils.native_rows import NativeRows

    rows = NativeRows(4, 100, 100, cuda)
    rows.zero_if_fresh()
    keys = torch.zeros((4, 128), dtype=torch.int16, device=cuda)
    budget = torch.zeros(4, dtype=torch.int32, device=cuda)
    prob = torch.zeros(4, dtype=torch.float32, device=cuda)

    def budget_args(start, rng, nb):
        return N.AdaptiveBudgetArgs(rows.as_struct(), keys.data_ptr(), 128, None, 0, 0, 0, N.dtype_code(torch.bfloat16),
                                    4, 1, 1.0, start, rng, nb, 0.1, 1.0, 1, 0, 0, budget.data_ptr(), prob.data_ptr(),
                                    None, N.stream_ptr(cuda))

    for bad in (budget_args(0, 1, 2), budget_args(50, 60, 2), budget_args(0, 100, 1)):
        with pytest.raises(ValueError):
            N.call("sah_adaptive_budget", bad)
    sample = N.AdaptiveSampleArgs(rows.as_struct(), budget.data_ptr(), prob.data_ptr(), N.dtype_code(torch.bfloat16),
                                  0, 100, 1, 1, 1, N.stream_ptr(cuda))
    with pytest.raises(N.NativeLibraryError, match="rows.w is NULL"):
        N.call("sah_adaptive_sample", sample)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_random_sampling_chain(cuda, dtype):
    """Sink + Local + RandomSampling: the final mask (weights included) equals the oracle's bit for bit, outputs
    within tolerance; a second call draws a different sample."""
    sa = _sa()
    B, Hq, Hkv, Lq, Lk, D = 2, 4, 2, 1, 700, 32
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, dtype, seed=11)
    cfgs = [sa.SinkMaskerConfig(sink_size=8), sa.LocalMaskerConfig(window_size=16), sa.RandomSamplingMaskerConfig(sampling_rate=0.1)]
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    ra.maskers[-1].seed = 99
    scaling = D ** -0.5
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, scaling, 0.0, sparse_meta_data={}, layer_idx=0)
    specs = [("sink", 8), ("local", 16), ("random", 0.1, 99, 0)]
    oo, ow, om = O.research_attention(specs, q, k, v, None, scaling)
    assert torch.equal(w.cpu() != 0, ow != 0)
    assert rel_err(out, oo) < TOL[dtype]
    assert (w.float().cpu() - ow.float()).abs().max().item() < (1e-6 if dtype == torch.float32 else 1e-2)
    out2, w2 = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, scaling, 0.0, sparse_meta_data={}, layer_idx=0)
    assert not torch.equal(w2 != 0, w != 0)


@pytest.mark.parametrize("base", ["hash", "pq"])
def test_composite_sampling_stacks(cuda, base):
    """The composite chains the reference ships builders for: Sink + Local + (HashAttention | PQCache) + AdaptiveSampling.
    Index sets bit-exact against the oracle given the kernels' signatures / codebook and budgets."""
    sa = _sa()
    dtype = torch.float32
    B, Hq, Hkv, Lq, Lk, D = 1, 4, 2, 1, 1200, 32
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, dtype, seed=13)
    cfgs = [sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=32)]
    specs = [("sink", 16), ("local", 32)]
    meta = {}
    if base == "hash":
        wts = _hat(sa, Hq, D, dtype, hidden=32)
        cfgs.append(sa.HashAttentionTopKMaskerConfig(heavy_size=40, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=32,
                                                     hat_mlp_activation="silu", hat_weights=wts))
    else:
        cfgs.append(sa.PQCacheConfig(heavy_size=40, pq_group_factor=4, pq_bits=4, kmeans_iter=4, init_offset=16, metric="euclidean"))
    cfgs.append(sa.AdaptiveSamplingMaskerConfig(base_rate_sampling=0.03, epsilon=0.1, delta=0.1, init_offset=16, local_offset=32))
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    ra.maskers[-1].seed = 7
    scaling = D ** -0.5
    out, w = ra.custom_attention(None, q.to(cuda), k.to(cuda), v.to(cuda), None, scaling, 0.0, sparse_meta_data=meta, layer_idx=0)
    torch.cuda.synchronize()
    state = {"budget": ra.maskers[-1].last_budget.cpu().long()}
    if base == "hash":
        state["key_sig"] = meta["key"][0].unpack(dtype).cpu()
        specs.append(("hash_topk", 40, wts[0], "silu"))
    else:
        cent = meta["pq_centroids"][0].cpu()
        book = meta["pq_codebook"][0].to_reference().cpu()
        specs.append(("pq_topk", 40, 16, cent, book))
    specs.append(("adaptive", 0.03, 0.1, 0.1, 16, 32, 7, 0))
    if base == "hash":
        # score with the kernel's own query signature too: recompute it through the masker
        qsig_codes = torch.empty((B * Hq * Lq, 2), dtype=torch.int32, device=cuda)
        ra.maskers[2]._hash(q.to(cuda), Hq, Hq, 0, Lq, 0, "query", qsig_codes, Lq, 0)
        from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.hashattention_top_k import (
            PackedSignatureCache)
        tmp = PackedSignatureCache.__new__(PackedSignatureCache)
        tmp.bits, tmp.n, tmp.codes = 32, Lq, qsig_codes.view(B, Hq, Lq, 2)
        state["query_sig"] = tmp.unpack(dtype).cpu()
    oo, ow, om = O.research_attention(specs, q, k, v, None, scaling, None, state)
    assert torch.equal(w.cpu() != 0, ow != 0)
    assert rel_err(out, oo) < TOL[dtype]


# ------------------------------------------------------------------------ logits from the scoring pass
def _key_scores(keys16, resid16, dtype):
    """fp32 (score, remainder) from the 16-bit score keys (the inverse of the order-preserving map) and the remainder
    words, both (rows, n) int16 tensors on the host."""
    k = keys16.to(torch.int32) & 0xFFFF
    bits = torch.where((k & 0x8000) != 0, k & 0x7FFF, (~k) & 0xFFFF).to(torch.int16)
    return bits.view(dtype).float(), resid16.view(dtype).float()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 8, 2, 1, 6000, 128, 900), (8, 32, 8, 1, 1500, 64, 300), (2, 4, 4, 2, 700, 128, 64)])
def test_attention_takes_its_logits_from_the_scoring_pass(cuda, dtype, shape):
    """`sah_qk_scores` with `resid_out`: the keys are unchanged and key + remainder reproduce the fp32 dot product to
    about 16 mantissa bits. `sah_sparse_attention` with `score_keys` / `score_resid`: the same output as from K (to the
    rounding of the 16-bit result), and K is not read at all - the call gives the same bits when K holds garbage."""
    from sparse_attention_hub_amd import _native as N
    from sparse_attention_hub_amd.sparse_attention.utils.mask_attention_utils import unit_inverse_weight

    B, Hq, Hkv, Lq, Lk, D, n_sel = shape
    q, k, v = make_qkv(B, Hq, Hkv, Lq, Lk, D, dtype, seed=31, outliers=True, device=cuda)
    n_rows = B * Hq * Lq
    pitch = (Lk + 63) // 64 * 64
    keys = torch.zeros((n_rows, pitch), dtype=torch.int16, device=cuda)
    keys_plain = torch.zeros_like(keys)
    resid = torch.zeros_like(keys)

    def score(keys_out, resid_out):
        N.call("sah_qk_scores", N.QkScoresArgs(
            q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), k.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
            None, 0, 0, 0, N.dtype_code(dtype), B, Hq, Hkv, Lq, Lk, D, keys_out.data_ptr(), pitch, N.stream_ptr(cuda),
            None if resid_out is None else resid_out.data_ptr()))

    score(keys, resid)
    score(keys_plain, None)
    torch.cuda.synchronize()
    assert torch.equal(keys, keys_plain)
    G = Hq // Hkv
    exact = torch.einsum("bhqd,bhkd->bhqk", q.double().cpu(), k.double().cpu().repeat_interleave(G, dim=1)).reshape(n_rows, Lk)
    s, rem = _key_scores(keys[:, :Lk].cpu(), resid[:, :Lk].cpu(), dtype)
    assert bool(torch.isfinite(s).all())
    scale = exact.abs().clamp_min(1.0)
    # the key alone is the score rounded to the tensor type (8 or 11 mantissa bits); with the remainder 2^-15 or better
    assert float(((s.double() - exact).abs() / scale).max()) > 2.0 ** -12
    assert float((((s + rem).double() - exact).abs() / scale).max()) < 2.0 ** -15

    g = torch.Generator().manual_seed(5)
    cols = torch.stack([torch.randperm(Lk, generator=g)[:n_sel] for _ in range(n_rows)]).to(torch.int32).to(cuda)
    cnt = torch.full((n_rows,), n_sel, dtype=torch.int32, device=cuda)
    cnt[0] = n_sel // 3
    w = (torch.rand((n_rows, n_sel), generator=g) * 0.9 + 0.1).to(cuda)
    bitmap = torch.zeros((n_rows, (Lk + 31) // 32), dtype=torch.int32, device=cuda)
    rows = N.Rows(cols.data_ptr(), cnt.data_ptr(), w.data_ptr(), bitmap.data_ptr(), n_rows, n_sel, Lk, (Lk + 31) // 32)
    work = torch.zeros((max(1, N.work_floats(n_rows, n_sel, D)),), dtype=torch.float32, device=cuda)
    sinks = torch.linspace(-1.0, 1.0, Hq, device=cuda)

    def attend(k_tensor, with_keys):
        out = torch.zeros((B, Lq, Hq, D), dtype=dtype, device=cuda)
        stats = torch.zeros((n_rows, 2), dtype=torch.float32, device=cuda)
        a = N.AttentionArgs(
            rows, q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
            k_tensor.data_ptr(), k_tensor.stride(0), k_tensor.stride(1), k_tensor.stride(2),
            v.data_ptr(), v.stride(0), v.stride(1), v.stride(2), None, 0, 0, 0, sinks.data_ptr(),
            N.dtype_code(dtype), B, Hq, Hkv, Lq, Lk, D, float(D ** -0.5), unit_inverse_weight(dtype), 0, 0, 0, 0, n_sel,
            out.data_ptr(), work.data_ptr(), work.numel(), None, stats.data_ptr(), N.stream_ptr(cuda))
        if with_keys:
            a.score_keys, a.score_resid, a.score_pitch = keys.data_ptr(), resid.data_ptr(), pitch
        N.call("sah_sparse_attention", a)
        torch.cuda.synchronize()
        return out, stats

    from_k, st_k = attend(k, False)
    from_keys, st_keys = attend(k, True)
    garbage = torch.full_like(k, 3.0)
    from_keys_no_k, _ = attend(garbage, True)
    wrong, _ = attend(garbage, False)
    assert torch.equal(from_keys, from_keys_no_k)             # K is not read
    assert rel_err(wrong, from_k) > 0.1                       # ... which the plain call would have noticed
    assert rel_err(from_keys, from_k) < (4e-3 if dtype == torch.bfloat16 else 1e-3)
    assert float((st_keys - st_k).abs().max() / st_k.abs().max()) < 1e-3


@pytest.mark.parametrize("case", ["one_per_row", "parts", "parts_keyed", "one_per_row_keyed", "not_fresh", "fallback_f32"])
def test_select_topk_attention_entry_point_against_the_two_calls(cuda, case):
    """`sah_select_topk_attention` through the C ABI (no plan in between): rows (column sets, counts, bitmap) and output
    of the one call against `sah_select_topk` followed by `sah_sparse_attention`, with one workgroup per row, with
    several (their partial results merged by the last arrival, the tickets left at zero), with the logits taken from the
    scoring pass, on rows that already hold sink and local columns, and where the one-kernel form does not apply."""
    from sparse_attention_hub_amd import _native as N
    from sparse_attention_hub_amd.sparse_attention.utils.mask_attention_utils import unit_inverse_weight
    from sparse_attention_hub_amd.sparse_attention.utils.native_rows import NativeRows

    dtype = torch.float32 if case == "fallback_f32" else torch.bfloat16
    B, Hq, Hkv, Lk, D = (8, 32, 8, 2500, 128) if case in ("one_per_row", "one_per_row_keyed", "not_fresh") else (1, 8, 2, 5000, 64)
    sink, window, k = 16, 48, 200
    keyed = case.endswith("keyed")
    fresh = case != "not_fresh"
    q, kk, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=17, outliers=True, device=cuda)
    n_rows = B * Hq
    pitch = (Lk + 63) // 64 * 64
    kdt = torch.int32 if dtype == torch.float32 else torch.int16
    keys = torch.zeros((n_rows, pitch), dtype=kdt, device=cuda)
    resid = torch.zeros_like(keys) if keyed else None
    N.call("sah_qk_scores", N.QkScoresArgs(
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), kk.data_ptr(), kk.stride(0), kk.stride(1), kk.stride(2),
        None, 0, 0, 0, N.dtype_code(dtype), B, Hq, Hkv, 1, Lk, D, keys.data_ptr(), pitch, N.stream_ptr(cuda),
        None if resid is None else resid.data_ptr()))
    cap = sink + window + k
    work = torch.zeros((max(1, N.work_floats(n_rows, cap, D)),), dtype=torch.float32, device=cuda)
    tickets = torch.zeros((n_rows,), dtype=torch.int32, device=cuda)
    excluded = 0  # the lowest key: active columns rank last

    def run(one_call):
        rows = NativeRows(n_rows, Lk, cap, cuda)
        if not fresh:
            N.call("sah_sink_local_indices", N.SinkLocalArgs(rows.as_struct(), 1, sink, window, 1, 0, N.stream_ptr(cuda)))
        sel = N.SelectTopkArgs(rows.as_struct(), keys.data_ptr(), pitch, 32 if dtype == torch.float32 else 16, Lk, 0, k, excluded,
                               1 if fresh else 0, sink if fresh else 0, window if fresh else 0, N.stream_ptr(cuda))
        out = torch.zeros((B, 1, Hq, D), dtype=dtype, device=cuda)
        att = N.AttentionArgs(
            rows.as_struct(), q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
            kk.data_ptr(), kk.stride(0), kk.stride(1), kk.stride(2), v.data_ptr(), v.stride(0), v.stride(1), v.stride(2),
            None, 0, 0, 0, None, N.dtype_code(dtype), B, Hq, Hkv, 1, Lk, D, float(D ** -0.5), unit_inverse_weight(dtype),
            0, 0, 0, 0, cap, out.data_ptr(), work.data_ptr(), work.numel(), None, None, N.stream_ptr(cuda))
        if keyed and one_call:
            att.score_keys, att.score_resid, att.score_pitch = keys.data_ptr(), resid.data_ptr(), pitch
        N.timing_enable(True)
        if one_call:
            rc = N.lib().sah_select_topk_attention(C.byref(sel), C.byref(att), C.c_void_p(tickets.data_ptr()))
            assert rc == 0, N.lib().sah_last_error()
        else:
            N.call("sah_select_topk", sel)
            N.call("sah_sparse_attention", att)
        torch.cuda.synchronize()
        names = set(N.timing_collect())
        N.timing_enable(False)
        return rows.cnt.cpu(), torch.sort(rows.cols.cpu(), dim=1).values, rows.bitmap.cpu(), out, names

    c1, s1, b1, o1, names1 = run(True)
    c2, s2, b2, o2, names2 = run(False)
    one_kernel = case not in ("fallback_f32",) and (fresh or n_rows >= 192)
    assert ("k_select16_attn" in names1) == one_kernel, names1
    assert "k_select16_attn" not in names2
    assert bool((c1 == cap).all()) and torch.equal(c1, c2)
    assert torch.equal(s1, s2) and torch.equal(b1, b2)          # skip_bitmap = 0: the bitmap rows are brought up to date
    assert int(tickets.abs().max()) == 0                         # the last arrival of every row has reset its ticket
    several = n_rows < 192
    if keyed or several:
        assert rel_err(o1, o2) < 4e-3
    else:
        assert torch.equal(o1, o2)


@pytest.mark.parametrize("case", ["bf16_decode_d64", "bf16_three_queries", "bf16_sinks_and_mask"])
def test_oracle_topk_chain_with_logits_from_the_scoring_pass(cuda, case):
    """Sink + Local + OracleTopK masker by masker (attention weights wanted, so no plan): the attention takes its logits
    from the scoring pass's keys and remainders - with head_dim 64, with several queries per head (mask rows =
    B x heads x queries), with sink logits, and with an additive mask (then the selection's scores carry the mask, are
    not shared, and the attention reads K as ever). Index sets, dense probabilities and outputs against the oracle.
    (bf16 only: in fp16 the reference's inverse-mask formula, 1 / (mask + 1e-6) * (mask != 0), is inf * 0 = NaN on every
    entry outside the mask, so there is nothing to compare with.)"""
    sa = _sa()
    cfgs = [sa.SinkMaskerConfig(sink_size=16), sa.LocalMaskerConfig(window_size=32), sa.OracleTopKConfig(heavy_size=0.05)]
    specs = [("sink", 16), ("local", 32), ("oracle_topk", 0.05)]
    if case == "bf16_decode_d64":
        _run_chain(cuda, cfgs, specs, 2, 8, 2, 1, 3000, 64, torch.bfloat16, seed=3)
    elif case == "bf16_three_queries":
        _run_chain(cuda, cfgs, specs, 1, 8, 4, 3, 2000, 128, torch.bfloat16, outliers=True, seed=4)
    else:
        am = torch.zeros(2, 1, 1, 2500)
        am[1, :, :, 700:900] = torch.finfo(torch.float32).min
        _run_chain(cuda, cfgs, specs, 2, 8, 2, 1, 2500, 128, torch.bfloat16, amask=am.to(torch.bfloat16),
                   sinks=torch.linspace(-1.0, 1.0, 8), outliers=True, seed=5)
