"""HuggingFace adapter: registration, sparse-mode switching and the prefill / question / decode loop on a tiny
random-weight Llama (no download). The CPU tests use a stand-in SparseAttention that computes dense attention with
HuggingFace's own eager kernel, which pins the adapter's plumbing: with it the loop must reproduce the plain model.
The GPU test runs the real kernels under the adapter against the CPU oracle plugged into the same model."""
import pytest
import torch

transformers = pytest.importorskip("transformers")


def _tiny_llama(dtype=torch.float32, layers=2, seed=0):
    from transformers import LlamaConfig, LlamaForCausalLM

    torch.manual_seed(seed)
    cfg = LlamaConfig(vocab_size=96, hidden_size=128, intermediate_size=256, num_hidden_layers=layers,
                      num_attention_heads=4, num_key_value_heads=2, head_dim=32, max_position_embeddings=1024)
    return LlamaForCausalLM(cfg).to(dtype).eval()


class _EagerStandIn:
    """Quacks like SparseAttention: dense attention through HuggingFace's eager kernel; records what it was given."""

    def __init__(self):
        self.calls = []

    def custom_attention(self, module, queries, keys, values, attention_mask, scaling, dropout, **kwargs):
        from transformers.models.llama.modeling_llama import eager_attention_forward

        self.calls.append((kwargs.get("layer_idx"), queries.shape[2], keys.shape[2], id(kwargs["sparse_meta_data"])))
        return eager_attention_forward(module, queries, keys, values, attention_mask, scaling=scaling, dropout=dropout)


def _registered_without_type_check(adapter):
    """Registration for a stand-in that is not a ResearchAttention instance."""
    from transformers.masking_utils import ALL_MASK_ATTENTION_FUNCTIONS, eager_mask
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    def ensure():
        if adapter._registered_attention_name is None:
            adapter._custom_attention_fn = adapter.get_custom_attention_function(adapter.sparse_attention)
            adapter._registered_attention_name = adapter._generate_unique_attention_name()
            ALL_ATTENTION_FUNCTIONS.register(adapter._registered_attention_name, adapter._custom_attention_fn)
            ALL_MASK_ATTENTION_FUNCTIONS.register(adapter._registered_attention_name, eager_mask)
        return adapter._registered_attention_name

    return ensure


def _adapter_with(model, stand_in):
    from sparse_attention_hub_amd.adapters import ModelAdapterHF

    adapter = ModelAdapterHF(model, None)
    adapter.sparse_attention = stand_in
    adapter._sparse_attention_available = True
    adapter._ensure_attention_registered = _registered_without_type_check(adapter)
    return adapter


def test_registration_is_unique_cached_and_cleaned_up():
    from sparse_attention_hub_amd.adapters import ModelAdapterHF
    from sparse_attention_hub_amd.sparse_attention import LocalMaskerConfig, ResearchAttentionConfig, SinkMaskerConfig
    from transformers.masking_utils import ALL_MASK_ATTENTION_FUNCTIONS
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    model = _tiny_llama()
    cfg = ResearchAttentionConfig(masker_configs=[SinkMaskerConfig(sink_size=4), LocalMaskerConfig(window_size=8)])
    adapter = ModelAdapterHF(model, cfg)
    assert adapter.sparse_attention.return_attention_weights is False
    name = adapter._ensure_attention_registered()
    assert name.startswith("sparse_attention_") and len(name) == len("sparse_attention_") + 8
    assert name in ALL_ATTENTION_FUNCTIONS.valid_keys() and name in ALL_MASK_ATTENTION_FUNCTIONS.valid_keys()
    assert adapter._ensure_attention_registered() == name                      # cached, not re-registered
    other = ModelAdapterHF(model, cfg)
    assert other._ensure_attention_registered() != name
    adapter._cleanup_attention_registration()
    assert name not in ALL_ATTENTION_FUNCTIONS.valid_keys() and name not in ALL_MASK_ATTENTION_FUNCTIONS.valid_keys()
    assert adapter._registered_attention_name is None
    other._cleanup_attention_registration()


def test_dense_only_adapter_refuses_sparse_mode():
    from sparse_attention_hub_amd.adapters import ModelAdapterHF

    adapter = ModelAdapterHF(_tiny_llama(), None)
    with pytest.raises(RuntimeError, match="Cannot enable sparse mode"):
        with adapter.enable_sparse_mode():
            pass
    with pytest.raises(RuntimeError, match="Cannot register attention function"):
        adapter._ensure_attention_registered()


def test_sparse_mode_switches_and_restores_the_attention_implementation():
    model = _tiny_llama()
    before = model.config._attn_implementation
    adapter = _adapter_with(model, _EagerStandIn())
    try:
        with adapter.enable_sparse_mode():
            assert model.config._attn_implementation == adapter._registered_attention_name
            with pytest.raises(ValueError, match="sparse_meta_data must be provided"):
                model(input_ids=torch.randint(0, 96, (1, 5)))
        assert model.config._attn_implementation == before
        # restored even when the body raises
        with pytest.raises(KeyError):
            with adapter.enable_sparse_mode():
                raise KeyError("boom")
        assert model.config._attn_implementation == before
    finally:
        adapter._cleanup_attention_registration()


@pytest.mark.parametrize("hybrid", [False, True])
def test_generation_loop_with_a_dense_stand_in_reproduces_the_plain_model(hybrid):
    model = _tiny_llama()
    g = torch.Generator().manual_seed(1)
    context = torch.randint(0, 96, (1, 40), generator=g)
    questions = [torch.randint(0, 96, (1, 6), generator=g), torch.randint(0, 96, (1, 3), generator=g)]
    stand_in = _EagerStandIn()
    adapter = _adapter_with(model, stand_in)
    adapter.hybrid = hybrid
    try:
        got = adapter.process_tokens(context, questions, max_new_tokens=5)
    finally:
        adapter._cleanup_attention_registration()
    # plain greedy decoding of the same prompts
    for q_tokens, answer in zip(questions, got):
        ids = torch.cat([context, q_tokens], dim=1)
        want = []
        with torch.no_grad():
            for _ in range(5):
                nxt = model(input_ids=ids).logits[0, -1].argmax()
                want.append(nxt)
                ids = torch.cat([ids, nxt.view(1, 1)], dim=1)
        assert torch.equal(answer, torch.stack(want))
    # every layer was called, with its index, and the question pass saw Lq > 1 unless fed token by token
    layers = {c[0] for c in stand_in.calls}
    assert layers == {0, 1}
    lqs = {c[1] for c in stand_in.calls}
    assert lqs == ({1} if hybrid else {1, 3, 6})
    # one sparse_meta_data dict per question, shared by all of its forward calls
    assert len({c[3] for c in stand_in.calls}) == 2


# --------------------------------------------------------------------------------------- GPU
class _OracleAttention:
    """The CPU oracle as a SparseAttention stand-in (test infrastructure): same masker chain, reference semantics."""

    def __init__(self, specs_for_layer):
        self.specs_for_layer = specs_for_layer
        self.state = {}

    def custom_attention(self, module, queries, keys, values, attention_mask, scaling, dropout, **kwargs):
        from oracle import reference_path as O

        layer = kwargs.get("layer_idx")
        st = self.state.setdefault(layer, {})
        st.pop("query_sig", None)
        out, _, _ = O.research_attention(self.specs_for_layer(layer), queries.cpu(), keys.cpu(), values.cpu(),
                                         None if attention_mask is None else attention_mask.cpu(), scaling, None, st)
        return out.to(queries.device), None


@pytest.mark.gpu
@pytest.mark.parametrize("chain", ["oracle_topk", "hash"])
def test_tiny_llama_through_the_adapter_matches_the_oracle(cuda, chain):
    """Question pass (Lq > 1, Local's future-clearing branch) and decode steps of a random tiny Llama through
    ALL_ATTENTION_FUNCTIONS: logits of the kernels against logits of the oracle plugged into the same model."""
    from sparse_attention_hub_amd.adapters import ModelAdapterHF
    from sparse_attention_hub_amd.sparse_attention import (
        HashAttentionTopKMaskerConfig, LocalMaskerConfig, OracleTopKConfig, ResearchAttentionConfig, SinkMaskerConfig)
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    model = _tiny_llama(torch.float32).to(cuda)
    cfgs = [SinkMaskerConfig(sink_size=4), LocalMaskerConfig(window_size=8)]
    if chain == "oracle_topk":
        cfgs.append(OracleTopKConfig(heavy_size=12))
        specs_for = lambda layer: [("sink", 4), ("local", 8), ("oracle_topk", 12)]
    else:
        wts = random_hat_weights(2, 4, 32, 16, 2, 32, dtype=torch.float32, seed=3)
        cfgs.append(HashAttentionTopKMaskerConfig(heavy_size=12, hat_bits=16, hat_mlp_layers=2, hat_mlp_hidden_size=32,
                                                  hat_mlp_activation="relu", hat_weights=wts))
        specs_for = lambda layer: [("sink", 4), ("local", 8), ("hash_topk", 12, wts[layer], "relu")]
    g = torch.Generator().manual_seed(2)
    context = torch.randint(0, 96, (1, 70), generator=g).to(cuda)
    question = torch.randint(0, 96, (1, 5), generator=g).to(cuda)
    steps = torch.randint(0, 96, (3,), generator=g).to(cuda)

    def run(adapter):
        meta = {}
        logits = []
        with torch.no_grad():
            ctx = model(context, past_key_values=None, use_cache=True, sparse_meta_data=meta)
            with adapter.enable_sparse_mode():
                out = model(input_ids=question, past_key_values=ctx.past_key_values, use_cache=True, sparse_meta_data=meta)
                logits.append(out.logits[0].float().cpu())
                past = out.past_key_values
                for t in steps:
                    out = model(input_ids=t.view(1, 1), past_key_values=past, use_cache=True, sparse_meta_data=meta)
                    logits.append(out.logits[0].float().cpu())
                    past = out.past_key_values
        adapter._cleanup_attention_registration()
        return logits

    ours = run(ModelAdapterHF(model, ResearchAttentionConfig(masker_configs=cfgs)))
    want = run(_adapter_with(model, _OracleAttention(specs_for)))
    for a, b in zip(ours, want):
        assert a.shape == b.shape
        assert ((a - b).norm() / b.norm()).item() < 1e-4


def _llama_shaped(cuda, layers=2, seed=0):
    """A random-weight Llama with Llama-3.1-8B's attention geometry (32 query / 8 KV heads of 128) and a narrow MLP."""
    from transformers import LlamaConfig, LlamaForCausalLM

    torch.manual_seed(seed)
    cfg = LlamaConfig(vocab_size=128, hidden_size=4096, intermediate_size=512, num_hidden_layers=layers,
                      num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=16384)
    return LlamaForCausalLM(cfg).to(torch.bfloat16).to(cuda).eval()


def _unpack_codes(codes):
    c = codes.cpu().long() & 0xFFFFFFFF
    shifts = torch.arange(32)
    pos = (c[..., 0].unsqueeze(-1) >> shifts) & 1
    nonzero = (c[..., 1].unsqueeze(-1) >> shifts) & 1
    return ((pos * 2 - 1) * nonzero).float()


@pytest.mark.gpu
def test_llama_shaped_decode_through_the_default_adapter_is_one_kernel_per_layer(cuda):
    """What HuggingFace hands the registered callable in a decode step is the eager mask, a (B, 1, 1, Lk) tensor that
    is all zeros when no sequence is padded (reference adapters/huggingface.py:227-275, :311-319). Through
    ModelAdapterHF with its default arguments a bf16 Llama-shaped stack (B = 8, 32 query / 8 KV heads of 128, 8192
    context keys, Sink + Local + HashAttention top-k) must run every decode layer-step as ONE launch of
    k_hash_decode_attn (plus one mask classification per forward pass), give the oracle's attention output on the
    tensors of every call HuggingFace makes, and select exactly the oracle's columns given the kernel's signatures.
    (Whole-model logits of two runs are not compared: with a random model a last-bit difference in one layer's output
    flips signature bits of the next layer's query, i.e. the comparison would be of two different selections.)"""
    from oracle import reference_path as O
    from sparse_attention_hub_amd import _native as N
    from sparse_attention_hub_amd.adapters import ModelAdapterHF
    from sparse_attention_hub_amd.sparse_attention import (
        HashAttentionTopKMaskerConfig, LocalMaskerConfig, ResearchAttentionConfig, SinkMaskerConfig)
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    B, Hq, D, n_ctx, layers = 8, 32, 128, 8192, 2
    sink, window, heavy = 128, 512, 1024
    model = _llama_shaped(cuda, layers)
    wts = random_hat_weights(layers, Hq, D, 32, 3, 128, dtype=torch.bfloat16, seed=5)
    cfgs = [SinkMaskerConfig(sink_size=sink), LocalMaskerConfig(window_size=window),
            HashAttentionTopKMaskerConfig(heavy_size=heavy, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                          hat_mlp_activation="silu", hat_weights=wts)]
    specs_for = lambda layer: [("sink", sink), ("local", window), ("hash_topk", heavy, wts[layer], "silu")]
    g = torch.Generator().manual_seed(4)
    context = torch.randint(0, 128, (B, n_ctx), generator=g).to(cuda)
    question = torch.randint(0, 128, (B, 4), generator=g).to(cuda)
    steps = torch.randint(0, 128, (5, B), generator=g).to(cuda)
    n_timed = 3

    def prefill(meta):
        past = None
        with torch.no_grad():
            for at in range(0, n_ctx, 2048):      # the model's own attention, in pieces
                out = model(context[:, at:at + 2048], past_key_values=past, use_cache=True, sparse_meta_data=meta)
                past = out.past_key_values
        return past

    def run(adapter, timed):
        meta, logits, launches = {}, [], None
        past = prefill(meta)
        with torch.no_grad(), adapter.enable_sparse_mode():
            out = model(input_ids=question, past_key_values=past, use_cache=True, sparse_meta_data=meta)
            logits.append(out.logits[:, -1].float().cpu())
            past = out.past_key_values
            for i, t in enumerate(steps):
                if timed and i == len(steps) - n_timed:
                    torch.cuda.synchronize()
                    N.timing_enable(True)
                out = model(input_ids=t.view(B, 1), past_key_values=past, use_cache=True, sparse_meta_data=meta)
                logits.append(out.logits[:, -1].float().cpu())
                past = out.past_key_values
            if timed:
                torch.cuda.synchronize()
                launches = N.timing_collect()
                N.timing_enable(False)
        adapter._cleanup_attention_registration()
        return logits, launches, meta

    adapter = ModelAdapterHF(model, ResearchAttentionConfig(masker_configs=cfgs))      # default arguments
    masker = adapter.sparse_attention.maskers[2]
    seen = {"calls": 0, "worst": 0.0}
    inner = adapter.sparse_attention.custom_attention

    def checked(module, queries, keys, values, attention_mask, scaling, dropout, **kw):
        """Every call HuggingFace makes (question pass and decode steps, both layers) against the oracle on the very
        tensors it was given, batch rows 0 and B - 1, scoring the kernels' own signature bits (a float MLP on the host
        may round a borderline output to the other side of zero; the MLP is compared bit by bit elsewhere)."""
        out = inner(module, queries, keys, values, attention_mask, scaling, dropout, **kw)
        layer, Lq = kw["layer_idx"], queries.shape[2]
        cache = kw["sparse_meta_data"]["key"][layer]
        qcodes = torch.empty((B * Hq * Lq, 2), dtype=torch.int32, device=cuda)
        masker._hash(queries, Hq, Hq, 0, Lq, layer, "query", qcodes, Lq, 0)
        qsig = _unpack_codes(qcodes).view(B, Hq, Lq, 32)
        n = min(cache.n, keys.shape[2])       # keys hashed so far; the rest sit inside the local window
        for b in (0, B - 1):
            state = {"key_sig": _unpack_codes(cache.codes[b:b + 1, :, :n]), "query_sig": qsig[b:b + 1]}
            oo, _, om = O.research_attention(specs_for(layer), queries[b:b + 1].cpu(), keys[b:b + 1].cpu(), values[b:b + 1].cpu(),
                                             attention_mask[b:b + 1].cpu(), scaling, state=state)
            got = out[0][b:b + 1].float().cpu()
            seen["worst"] = max(seen["worst"], ((got - oo.float()).norm() / oo.float().norm()).item())
            seen["last"] = (layer, b, om, attention_mask, keys.shape[2])
        seen["calls"] += 1
        return out

    adapter.sparse_attention.custom_attention = checked
    ours, launches, meta = run(adapter, True)
    assert seen["calls"] == layers * (1 + len(steps)) and len(ours) == 1 + len(steps)
    assert seen["worst"] < 2e-2, seen["worst"]
    assert set(launches) - {"k_hash_sig_small_mfma", "k_hash_sig_gemv"} == {"k_hash_decode_attn", "k_amask_classify"}, launches
    assert launches["k_hash_decode_attn"][0] == n_timed * layers and launches["k_amask_classify"][0] == n_timed, launches
    # the stand-alone signature kernel above is the check's own (the query signatures it hands the oracle)
    assert all(launches[n][0] == n_timed * layers for n in launches if n.startswith("k_hash_sig")), launches

    # the last layer-step: what HuggingFace passed, and the columns the kernel selected for it
    layer, b, om, amask, Lk = seen["last"]
    assert layer == layers - 1 and b == B - 1 and tuple(amask.shape) == (B, 1, 1, Lk) and not bool(amask.any())
    plan = next(iter(adapter.sparse_attention._plans.values()))
    total = sink + window + heavy
    assert bool((plan.cnt.cpu() == total).all())
    member = torch.zeros((B * Hq, Lk), dtype=torch.bool, device=cuda)
    member.scatter_(1, plan.cols[:, :total].long(), True)
    member = member.cpu().view(B, Hq, Lk)
    assert torch.equal(member[b], om.to_dense()[0, :, 0] != 0), "selected sets differ"


@pytest.mark.gpu
def test_padded_batch_decode_through_the_default_adapter_matches_the_oracle(cuda):
    """A left-padded batch: the eager mask hides the padding columns with finfo.min, so it is not all zeros and must
    be honoured by the top-k scores and by the attention logits (hashattention_top_k.py:367-368,
    utils/mask_attention_utils.py:221-225)."""
    from sparse_attention_hub_amd.adapters import ModelAdapterHF
    from sparse_attention_hub_amd.sparse_attention import (
        LocalMaskerConfig, OracleTopKConfig, ResearchAttentionConfig, SinkMaskerConfig)

    model = _tiny_llama(torch.float32).to(cuda)
    cfgs = [SinkMaskerConfig(sink_size=4), LocalMaskerConfig(window_size=8), OracleTopKConfig(heavy_size=12)]
    specs_for = lambda layer: [("sink", 4), ("local", 8), ("oracle_topk", 12)]
    g = torch.Generator().manual_seed(6)
    B, n_ctx, pad = 2, 60, 9
    context = torch.randint(0, 96, (B, n_ctx), generator=g).to(cuda)
    amask = torch.ones(B, n_ctx, dtype=torch.long, device=cuda)
    amask[1, :pad] = 0                                                 # row 1 starts with 9 padding tokens
    steps = torch.randint(0, 96, (3, B), generator=g).to(cuda)
    seen = []

    def run(adapter, record):
        meta, logits, am = {}, [], amask
        with torch.no_grad():
            ctx = model(context, attention_mask=am, past_key_values=None, use_cache=True, sparse_meta_data=meta)
            past = ctx.past_key_values
            with adapter.enable_sparse_mode():
                for t in steps:
                    am = torch.cat([am, torch.ones(B, 1, dtype=torch.long, device=cuda)], dim=1)
                    out = model(input_ids=t.view(B, 1), attention_mask=am, past_key_values=past, use_cache=True,
                                sparse_meta_data=meta)
                    logits.append(out.logits[:, -1].float().cpu())
                    past = out.past_key_values
        adapter._cleanup_attention_registration()
        return logits

    adapter = ModelAdapterHF(model, ResearchAttentionConfig(masker_configs=cfgs))
    inner = adapter.sparse_attention.custom_attention

    def recording(module, queries, keys, values, attention_mask, scaling, dropout, **kw):
        seen.append(attention_mask)
        return inner(module, queries, keys, values, attention_mask, scaling, dropout, **kw)

    adapter.sparse_attention.custom_attention = recording
    ours = run(adapter, True)
    assert all(m is not None and float(m[1, 0, 0, :pad].max()) < -1e30 and not bool(m[0].any()) for m in seen)
    want = run(_adapter_with(model, _OracleAttention(specs_for)), False)
    for a, b in zip(ours, want):
        assert ((a - b).norm() / b.norm()).item() < 1e-4
