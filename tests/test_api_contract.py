"""The plug-in contract of the ResearchAttention path, without a GPU: class hierarchy, registry, factories, config
validation and error texts as the reference's own unit tests state them
(tests/unit/sparse_attention/test_configs_and_factories.py, research_attention/test_base.py,
research_attention/maskers/test_base.py, maskers/fixed/test_base.py, maskers/sampling/test_base.py, and the config
checks of maskers/fixed/implementations/test_basic_fixed.py, test_pq_top_k.py and
maskers/sampling/test_adaptive_sampling.py, test_implementations.py). Nothing here launches a kernel."""
import pytest
import torch

import sparse_attention_hub_amd.sparse_attention as sa
from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.base import AttentionTensorDimensions

HAT = dict(heavy_size=8, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=64, hat_mlp_activation="silu", hat_weights={})
ADAPTIVE = dict(base_rate_sampling=0.1, epsilon=0.25, delta=0.25, init_offset=4, local_offset=4)
PQ = dict(heavy_size=10, pq_group_factor=2, pq_bits=4, kmeans_iter=5, init_offset=4, metric="euclidean")


def test_class_hierarchy():
    # maskers/fixed/test_base.py:101-128, maskers/sampling/test_base.py:54-63, research_attention/test_base.py:70-87
    assert issubclass(sa.FixedMasker, sa.ResearchMasker) and issubclass(sa.TopKMasker, sa.FixedMasker)
    assert issubclass(sa.SamplingMasker, sa.ResearchMasker)
    for cls in (sa.SinkMasker, sa.LocalMasker, sa.CausalMasker):
        assert issubclass(cls, sa.FixedMasker)
    for cls in (sa.OracleTopK, sa.HashAttentionTopKMasker, sa.PQCache):
        assert issubclass(cls, sa.TopKMasker)
    for cls in (sa.RandomSamplingMasker, sa.AdaptiveSamplingMasker):
        assert issubclass(cls, sa.SamplingMasker)
    assert issubclass(sa.FixedMaskerConfig, sa.MaskerConfig) and issubclass(sa.TopKMaskerConfig, sa.FixedMaskerConfig)
    assert issubclass(sa.SamplingMaskerConfig, sa.MaskerConfig)
    for cfg in (sa.OracleTopKConfig, sa.HashAttentionTopKMaskerConfig, sa.PQCacheConfig):
        assert issubclass(cfg, sa.TopKMaskerConfig)
    assert issubclass(sa.ResearchAttention, sa.SparseAttention)
    assert issubclass(sa.ResearchAttentionConfig, sa.SparseAttentionConfig)


@pytest.mark.parametrize("config,cls", [
    (lambda: sa.LocalMaskerConfig(window_size=10), sa.LocalMasker),
    (lambda: sa.SinkMaskerConfig(sink_size=5), sa.SinkMasker),
    (lambda: sa.OracleTopKConfig(heavy_size=10), sa.OracleTopK),
    (lambda: sa.PQCacheConfig(**PQ), sa.PQCache),
    (lambda: sa.HashAttentionTopKMaskerConfig(**HAT), sa.HashAttentionTopKMasker),
    (lambda: sa.RandomSamplingMaskerConfig(sampling_rate=0.5), sa.RandomSamplingMasker),
    (lambda: sa.AdaptiveSamplingMaskerConfig(**ADAPTIVE), sa.AdaptiveSamplingMasker),
])
def test_registry_maps_every_config_to_its_masker(config, cls):
    # maskers/test_base.py:102-266: ResearchMasker.create_masker_from_config(config) -> instance of the masker, holding the config
    cfg = config()
    m = sa.ResearchMasker.create_masker_from_config(cfg)
    assert type(m) is cls and m.config is cfg
    # the class's own factory gives the same, and refuses a config of another masker ("Invalid config type")
    assert type(cls.create_from_config(cfg)) is cls
    other = sa.SinkMaskerConfig(sink_size=1) if cls is not sa.SinkMasker else sa.LocalMaskerConfig(window_size=1)
    with pytest.raises(ValueError, match="Invalid config type"):
        cls.create_from_config(other)
    assert sa.MaskerRegistry.get_masker_class(type(cfg)) is cls


def test_unregistered_config_is_refused():
    class Stray(sa.MaskerConfig):
        pass

    with pytest.raises(ValueError, match="No masker class registered for config type"):
        sa.ResearchMasker.create_masker_from_config(Stray())


def test_research_attention_from_maskers_and_from_config():
    # research_attention/test_base.py:29-68, test_configs_and_factories.py:238-307
    cfgs = [sa.SinkMaskerConfig(sink_size=4), sa.LocalMaskerConfig(window_size=8), sa.OracleTopKConfig(heavy_size=0.1)]
    ra = sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs))
    assert [type(m) for m in ra.maskers] == [sa.SinkMasker, sa.LocalMasker, sa.OracleTopK]
    direct = sa.ResearchAttention(sa.SparseAttentionConfig(), [sa.SinkMasker.create_from_config(cfgs[0])])
    assert len(direct.maskers) == 1
    # the generic factory routes by config type (sparse_attention/base.py)
    routed = sa.SparseAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=cfgs[:1]))
    assert isinstance(routed, sa.ResearchAttention)
    with pytest.raises(TypeError):
        sa.ResearchAttention.create_from_config(sa.SparseAttentionConfig())


def test_at_most_one_sampling_masker():
    # research_attention/test_base.py:89-189
    text = "Only one sampling masker supported for efficiency; consider implementing all sampling logic in one masker"
    local = sa.LocalMasker.create_from_config(sa.LocalMaskerConfig(window_size=10))
    rnd = sa.RandomSamplingMasker.create_from_config(sa.RandomSamplingMaskerConfig(sampling_rate=0.5))
    ada = sa.AdaptiveSamplingMasker.create_from_config(sa.AdaptiveSamplingMaskerConfig(**ADAPTIVE))
    assert len(sa.ResearchAttention(sa.SparseAttentionConfig(), [local, rnd]).maskers) == 2
    assert len(sa.ResearchAttention(sa.SparseAttentionConfig(), [local]).maskers) == 1
    with pytest.raises(ValueError, match=text):
        sa.ResearchAttention(sa.SparseAttentionConfig(), [rnd, ada])
    with pytest.raises(ValueError, match=text):
        sa.ResearchAttention.create_from_config(sa.ResearchAttentionConfig(masker_configs=[
            sa.RandomSamplingMaskerConfig(sampling_rate=0.5), sa.AdaptiveSamplingMaskerConfig(**ADAPTIVE)]))


def test_fixed_masker_config_checks():
    # test_basic_fixed.py:320, :534
    with pytest.raises(ValueError, match="window_size must be > 0, got 0"):
        sa.LocalMaskerConfig(window_size=0)
    with pytest.raises(ValueError, match="sink_size must be > 0, got 0"):
        sa.SinkMaskerConfig(sink_size=0)
    assert sa.LocalMaskerConfig(window_size=0.25).window_size == 0.25 and sa.SinkMaskerConfig(sink_size=3).sink_size == 3


@pytest.mark.parametrize("field,value,text", [
    ("pq_group_factor", 0, "pq_group_factor must be > 0"), ("pq_group_factor", -1, "pq_group_factor must be > 0"),
    ("pq_bits", 0, "pq_bits must be > 0"), ("kmeans_iter", 0, "kmeans_iter must be > 0"),
    ("init_offset", -1, "init_offset must be >= 0"), ("metric", "cosine", "metric must be 'euclidean' or 'ip'"),
    ("metric", "", "metric must be 'euclidean' or 'ip'"),
])
def test_pq_config_checks(field, value, text):
    # test_pq_top_k.py:882-953
    with pytest.raises(ValueError, match=text):
        sa.PQCacheConfig(**{**PQ, field: value})


def test_pq_masker_input_checks():
    # test_pq_top_k.py:974-986
    m = sa.PQCache.create_from_config(sa.PQCacheConfig(**PQ))
    with pytest.raises(ValueError, match="sparse_meta_data cannot be None"):
        m._validate_inputs(None, {"layer_idx": 0})
    with pytest.raises(ValueError, match="layer_idx must be provided"):
        m._validate_inputs({}, {})
    with pytest.raises(ValueError, match="layer_idx must be provided"):
        m._validate_inputs({}, {"other_key": "value"})
    assert m._validate_inputs({}, {"layer_idx": 3}) == 3


@pytest.mark.parametrize("change,text", [
    (dict(base_rate_sampling=1.5), r"base_rate_sampling must be in \[0, 1\) if float"),
    (dict(base_rate_sampling=-1), "base_rate_sampling must be non-negative if int"),
    (dict(epsilon=0.0), r"epsilon must be in \(0, 1\)"), (dict(epsilon=1.0), r"epsilon must be in \(0, 1\)"),
    (dict(delta=0.0), r"delta must be in \(0, 1\)"), (dict(delta=1.0), r"delta must be in \(0, 1\)"),
    (dict(init_offset=-1), "init_offset must be non-negative"), (dict(local_offset=-1), "local_offset must be non-negative"),
])
def test_adaptive_sampling_config_checks(change, text):
    # test_adaptive_sampling.py:65-147
    with pytest.raises(ValueError, match=text):
        sa.AdaptiveSamplingMaskerConfig(**{**ADAPTIVE, **change})


@pytest.mark.parametrize("rate", [0.0, -0.1, 1.1, 2.0])
def test_random_sampling_config_checks(rate):
    # test_implementations.py:66-69, :230-233
    with pytest.raises(ValueError, match=rf"sampling_rate must be in range \(0, 1\], got {rate}"):
        sa.RandomSamplingMaskerConfig(sampling_rate=rate)


def test_effective_sizes_follow_the_reference_rule():
    # maskers/base.py: an int is an absolute count, a float a fraction of the key length (truncated)
    m = sa.OracleTopK.create_from_config(sa.OracleTopKConfig(heavy_size=0.05))
    assert m._calculate_effective_size(0.05, 32768) == 1638 and m._calculate_effective_size(7, 100) == 7
    assert m._calculate_effective_size(0.02, 131072) == 2621
    dims = AttentionTensorDimensions(batch_size=2, num_heads=4, seq_len_queries=1, seq_len_keys=9)
    assert (dims.batch_size, dims.num_heads, dims.seq_len_queries, dims.seq_len_keys) == (2, 4, 1, 9)


def test_full_mask_needs_no_device():
    # utils/mask.py: a full mask is a flag, not a tensor; maskers return it unchanged (basic_fixed.py:31-33 and peers)
    full = sa.Mask.create_full_mask((1, 2, 1, 8), torch.float32, "cpu")
    assert full.is_full_mask() and full.get_density() == 1.0
    empty = sa.Mask.create_empty_mask((1, 2, 1, 8), torch.float32, "cpu")
    assert empty.is_empty and not empty.is_full and empty.get_density() == 0.0
