"""CPU tests of the adaptive-sampling restatement and of the masker's host logic.

Known answers come from the reference's own unit tests
(tests/unit/sparse_attention/research_attention/maskers/sampling/test_adaptive_sampling.py):
sampling range (:207-250), base sample count (:252-272), std estimate against the true
std (:274-311), the budget reaching the requested failure rate on N(0,1) data (:313-357),
early exits (:359-453) and config validation (:14-148). The index streams themselves are
generator-specific in the reference; the Philox generator the kernels use is pinned by the
known-answer vectors published with the algorithm (Random123, kat_vectors).
"""
import numpy as np
import pytest
import torch

from oracle import reference_path as O


def _sa():
    import sparse_attention_hub_amd.sparse_attention as sa

    return sa


# ----------------------------------------------------------------------------- Philox
@pytest.mark.parametrize("ctr,key,out", [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
])
def test_philox4x32_10_known_answers(ctr, key, out):
    got = O.philox4x32_10(np.array(ctr, dtype=np.uint64), key)
    assert tuple(int(x) for x in got) == out


def test_philox_columns_are_uniform_on_the_range_and_reproducible():
    a = O.philox_columns(seed=7, offset=3, row=5, n=40000, start=10, rng=50)
    b = O.philox_columns(seed=7, offset=3, row=5, n=40000, start=10, rng=50)
    assert torch.equal(a, b)
    assert int(a.min()) == 10 and int(a.max()) == 59
    counts = torch.bincount(a - 10, minlength=50).double()
    chi2 = float(((counts - 800.0) ** 2 / 800.0).sum())
    assert chi2 < 100.0  # 49 degrees of freedom: P(chi2 > 100) ~ 2e-5
    # a prefix of a longer stream is the shorter stream; rows, offsets and seeds decorrelate
    assert torch.equal(O.philox_columns(7, 3, 5, 17, 10, 50), a[:17])
    for other in (O.philox_columns(8, 3, 5, 4000, 10, 50), O.philox_columns(7, 4, 5, 4000, 10, 50),
                  O.philox_columns(7, 3, 6, 4000, 10, 50)):
        assert float((other == a[:4000]).double().mean()) < 0.05


# ------------------------------------------------------------------------ closed forms
def test_sampling_range_known_answers():
    assert O.adaptive_sampling_range(16, 0, 0) == (0, 16, 16)
    assert O.adaptive_sampling_range(16, 2, 3) == (2, 13, 11)
    assert O.adaptive_sampling_range(16, 10, 10) == (10, 6, -4)
    assert O.adaptive_sampling_range(1000, 0.1, 0.2) == (100, 800, 700)


def test_base_count_known_answers():
    assert O.adaptive_base_count(0.1, 1000) == 100
    assert O.adaptive_base_count(5, 16) == 5
    assert O.adaptive_base_count(0.01, 50) == 2
    assert O.adaptive_base_count(1, 50) == 2


@pytest.mark.parametrize("epsilon,delta", [(0.2, 0.2), (0.25, 0.25), (0.5, 0.5), (0.2, 0.1)])
def test_budget_reaches_the_requested_failure_rate(epsilon, delta):
    """The reference's statistical check of the budget formula on N(0,1) data (:313-357)."""
    from statistics import NormalDist

    g = torch.Generator().manual_seed(1)
    n = 100000
    data = torch.randn(1, n, generator=g)
    static = 10000
    true_den = data.sum(dim=-1, keepdim=True) + static
    budget = int(O.adaptive_budget_formula(torch.ones(1, 1), true_den, n, epsilon,
                                           float(NormalDist().inv_cdf(1 - delta))).item())
    misses, runs = 0, 600
    for _ in range(runs):
        idx = torch.randperm(n, generator=g)[:budget]
        est = (data[:, idx].sum(dim=-1) * (n / budget)).item() + static
        misses += float((true_den.item() - est) > true_den.item() * epsilon)
    torch.testing.assert_close(misses / runs, delta, rtol=0.2, atol=0.05)


def test_budget_formula_against_hand_arithmetic():
    # (ppf * sigma * n / (eps * D))^2 with sigma=0.5, n=1000, eps=0.1, D=200, ppf=2 -> (1000/20)^2 = 2500 -> clamp 1000
    b = O.adaptive_budget_formula(torch.tensor([[0.5]]), torch.tensor([[200.0]]), 1000, 0.1, 2.0)
    assert int(b) == 1000
    b = O.adaptive_budget_formula(torch.tensor([[0.05]]), torch.tensor([[400.0]]), 1000, 0.1, 2.0)
    assert int(b) == 6  # (100 / 40)^2 = 6.25, truncated
    b = O.adaptive_budget_formula(torch.tensor([[1e-9]]), torch.tensor([[400.0]]), 1000, 0.1, 2.0)
    assert int(b) == 1


def test_std_estimate_and_denominators_of_adaptive_budget():
    """sigma is the unbiased std over the draws (duplicates included); the sampled denominator counts
    every distinct drawn column once at weight 1/(nb/n + 1e-6); static comes from the previous mask."""
    B, H, Lq, Lk = 1, 2, 1, 64
    g = torch.Generator().manual_seed(3)
    expw = torch.rand(B, H, Lq, Lk, generator=g)
    prev = O.sink(O.OMask.empty((B, H, Lq, Lk), torch.float32), 4)
    base = torch.tensor([[[[10, 11, 11, 20, 33]], [[40, 40, 40, 41, 5]]]])
    start, end = 4, 60
    n, nb = end - start, 5
    budget, prob = O.adaptive_budget(prev, expw, base, start, end, epsilon=0.3, delta=0.3)
    from statistics import NormalDist

    ppf = NormalDist().inv_cdf(0.7)
    for h in range(H):
        e = expw[0, h, 0].double()
        draws = base[0, h, 0]
        sigma = e[draws].std(unbiased=True)
        static = e[:4].sum() / (1 + 1e-6)
        sampled = e[torch.unique(draws)].sum() / (nb / n + 1e-6)
        want = (ppf * sigma * n / (0.3 * (static + sampled))) ** 2
        want = int(min(max(float(want), 1.0), n))
        want = min(max(want, nb), n)
        assert int(budget[0, h, 0, 0]) == want
        assert float(prob[0, h, 0, 0]) == pytest.approx(want / n, rel=1e-6)


def test_adaptive_merge_keeps_active_weights_and_collapses_duplicates():
    shape = (1, 1, 2, 12)
    prev = O.local(O.sink(O.OMask.empty(shape, torch.float32), 2), 2)
    draws = [torch.tensor([3, 3, 5, 0]), torch.tensor([4, 11, 4])]
    m = O.adaptive_merge(prev, draws, torch.tensor([0.25, 0.5]))
    d = m.to_dense()[0, 0]
    pd = prev.to_dense()[0, 0]
    assert torch.equal(d[0] != 0, (pd[0] != 0) | torch.tensor([c in (3, 5, 0) for c in range(12)]))
    assert d[0, 3] == 0.25 and d[0, 5] == 0.25 and d[0, 0] == 1.0  # column 0 was a sink entry: clamp(1 + p)
    assert d[1, 4] == 0.5 and d[1, 11] == 1.0
    assert float(d[0].sum()) == pytest.approx(float(pd[0].sum()) + 0.5)


def test_adaptive_sampling_composition_properties():
    """Rows hold the previous entries plus exactly the distinct budgeted draws, all inside the range, with the
    row's probability as weight (the sampler properties of test_mask_attention_utils.py:137-363)."""
    B, H, Lq, Lk, D = 1, 2, 1, 300, 8
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, H, Lq, D, generator=g)
    k = torch.randn(B, H, Lk, D, generator=g)
    prev = O.local(O.sink(O.OMask.empty((B, H, Lq, Lk), torch.float32), 8), 16)
    m, budget, prob = O.adaptive_sampling(prev, q, k, None, D ** -0.5, 0.05, 0.2, 0.2, 8, 16, seed=11, offset=4)
    start, end, n = 8, Lk - 16, Lk - 24
    nb = int(0.05 * n)
    d = m.to_dense()
    for h in range(H):
        b = int(budget[0, h, 0, 0])
        assert nb <= b <= n
        draws = O.philox_columns(11, 5, h, b, start, n)
        new = d[0, h, 0, start:end]
        assert int((new != 0).sum()) == torch.unique(draws).numel()
        assert torch.all(new[new != 0] == prob[0, h, 0, 0])
        assert torch.all(d[0, h, 0, :start] == 1) and torch.all(d[0, h, 0, end:] == 1)
    # full previous mask and a zero rate leave the mask alone; a range below 2 gives a full mask
    full = O.OMask.full((B, H, Lq, Lk), torch.float32)
    assert O.adaptive_sampling(full, q, k, None, 1.0, 0.05, 0.2, 0.2, 0, 0, 0, 0)[0] is full
    assert O.adaptive_sampling(prev, q, k, None, 1.0, 0, 0.2, 0.2, 0, 0, 0, 0)[0] is prev
    assert O.adaptive_sampling(prev, q, k, None, 1.0, 0.05, 0.2, 0.2, 150, 149, 0, 0)[0].kind == "full"


# ----------------------------------------------------------------- host logic of the masker
def _cfg(**kw):
    base = dict(base_rate_sampling=0.1, epsilon=0.1, delta=0.05, init_offset=0, local_offset=0)
    base.update(kw)
    return _sa().AdaptiveSamplingMaskerConfig(**base)


@pytest.mark.parametrize("kw,msg", [
    (dict(base_rate_sampling=1.0), r"base_rate_sampling must be in \[0, 1\) if float"),
    (dict(base_rate_sampling=-0.1), r"base_rate_sampling must be in \[0, 1\) if float"),
    (dict(base_rate_sampling=-1), "base_rate_sampling must be non-negative if int"),
    (dict(base_rate_sampling="0.1"), "base_rate_sampling must be int or float"),
    (dict(epsilon=0.0), r"epsilon must be in \(0, 1\)"),
    (dict(epsilon=1.0), r"epsilon must be in \(0, 1\)"),
    (dict(delta=0.0), r"delta must be in \(0, 1\)"),
    (dict(delta=1.5), r"delta must be in \(0, 1\)"),
    (dict(init_offset=-1), "init_offset must be non-negative if int"),
    (dict(init_offset=1.5), r"init_offset must be in \[0, 1\] if float"),
    (dict(local_offset=-1), "local_offset must be non-negative if int"),
    (dict(local_offset=-0.5), r"local_offset must be in \[0, 1\] if float"),
    (dict(local_offset="x"), "local_offset must be int or float"),
])
def test_config_validation_messages(kw, msg):
    with pytest.raises(ValueError, match=msg):
        _cfg(**kw)


def test_masker_construction_and_helpers():
    sa = _sa()
    cfg = _cfg()
    m = sa.ResearchMasker.create_masker_from_config(cfg)
    assert isinstance(m, sa.AdaptiveSamplingMasker) and isinstance(m, sa.SamplingMasker)
    assert (m.base_rate_sampling, m.epsilon, m.delta, m.init_offset, m.local_offset) == (0.1, 0.1, 0.05, 0, 0)
    assert m.delta_ppf == pytest.approx(1.6448536269514722, rel=1e-12)  # scipy.stats.norm.ppf(0.95)
    assert m._get_sampling_range(16) == (0, 16, 16)
    assert sa.AdaptiveSamplingMasker(_cfg(init_offset=2, local_offset=3))._get_sampling_range(16) == (2, 13, 11)
    bad = sa.AdaptiveSamplingMasker(_cfg(init_offset=10, local_offset=10))
    assert bad._get_sampling_range(16)[2] == -4 and bad.should_return_full_mask(-4) is True
    assert sa.AdaptiveSamplingMasker(_cfg(init_offset=0.1, local_offset=0.2))._get_sampling_range(1000) == (100, 800, 700)
    assert m._get_base_sample_count(1000) == 100
    assert sa.AdaptiveSamplingMasker(_cfg(base_rate_sampling=5))._get_base_sample_count(16) == 5
    assert sa.AdaptiveSamplingMasker(_cfg(base_rate_sampling=0.01))._get_base_sample_count(50) == 2
    with pytest.raises(ValueError, match="Invalid config type"):
        sa.AdaptiveSamplingMasker.create_from_config(sa.SinkMaskerConfig(sink_size=1))


def test_masker_early_exits_need_no_device():
    sa = _sa()
    shape = (2, 4, 8, 16)
    q = torch.randn(2, 4, 8, 32)
    k = torch.randn(2, 4, 16, 32)
    full = sa.Mask.create_full_mask(shape, torch.float32, torch.device("cpu"))
    m = sa.AdaptiveSamplingMasker(_cfg())
    assert m.add_mask(k, q, k, None, 1.0, 0.0, {}, full) is full
    empty = sa.Mask.create_empty_mask(shape, torch.float32, torch.device("cpu"))
    for rate in (0, 0.0):
        z = sa.AdaptiveSamplingMasker(_cfg(base_rate_sampling=rate))
        out = z.add_mask(k, q, k, None, 1.0, 0.0, {}, empty)
        assert out is empty and out.is_empty
    tiny = sa.AdaptiveSamplingMasker(_cfg(init_offset=10, local_offset=10))
    assert tiny.add_mask(k, q, k, None, 1.0, 0.0, {}, empty).is_full_mask()


def test_only_one_sampling_masker_per_chain():
    sa = _sa()
    with pytest.raises(ValueError, match="Only one sampling masker supported"):
        sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[_cfg(), _cfg()]))


# ----------------------------------------------------------------- random sampling
def test_random_sampling_oracle_and_masker_host_logic():
    """int(rate * n_keys) draws per row on [0, n_keys), weight = rate, clamp(previous + rate); full mask untouched;
    config validation of the reference (random_sampling.py:38-44)."""
    sa = _sa()
    shape = (1, 2, 1, 50)
    prev = O.sink(O.OMask.empty(shape, torch.float32), 3)
    m = O.random_sampling(prev, 0.2, seed=5, offset=0)
    d = m.to_dense()
    for h in range(2):
        draws = O.philox_columns(5, 0, h, 10, 0, 50)
        assert int(draws.min()) >= 0 and int(draws.max()) < 50
        new = set(draws.tolist()) - {0, 1, 2}
        assert set(torch.nonzero(d[0, h, 0]).flatten().tolist()) == new | {0, 1, 2}
        for c in new:
            assert float(d[0, h, 0, c]) == pytest.approx(0.2)
        assert torch.all(d[0, h, 0, :3] == 1.0)
    full = O.OMask.full(shape, torch.float32)
    assert O.random_sampling(full, 0.2, 5, 0) is full
    for bad in (0.0, -0.1, 1.5):
        with pytest.raises(ValueError, match=r"sampling_rate must be in range \(0, 1\]"):
            sa.RandomSamplingMaskerConfig(sampling_rate=bad)
    masker = sa.ResearchMasker.create_masker_from_config(sa.RandomSamplingMaskerConfig(sampling_rate=0.5))
    assert isinstance(masker, sa.RandomSamplingMasker) and masker.sampling_rate == 0.5
    fm = sa.Mask.create_full_mask(shape, torch.float32, torch.device("cpu"))
    q = torch.randn(1, 2, 1, 8)
    k = torch.randn(1, 2, 50, 8)
    assert masker.add_mask(k, q, k, None, 1.0, 0.0, {}, fm) is fm
    tiny = sa.RandomSamplingMasker(sa.RandomSamplingMaskerConfig(sampling_rate=0.01))
    em = sa.Mask.create_empty_mask(shape, torch.float32, torch.device("cpu"))
    assert tiny.add_mask(k, q, k, None, 1.0, 0.0, {}, em) is em   # int(0.01 * 50) = 0 draws
    with pytest.raises(ValueError, match="Invalid config type"):
        sa.RandomSamplingMasker.create_from_config(sa.SinkMaskerConfig(sink_size=1))
