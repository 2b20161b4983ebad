#!/usr/bin/env python3
"""Decode layer-step benchmark of the MI355X ResearchAttention path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1|2|3|4|5]

A step is one `ResearchAttention.custom_attention` call with one query token on a warm
cache (hash signatures / PQ codes of all earlier keys already built, one new key appended
per step), on synthetic inputs that are resident in HBM before the timed region. Default
workload: headline configuration 3, the one the headline target is quoted on (Sink 128 + Local 512
+ HashAttention top-2048, batch 8, 32 query / 8 KV heads, head_dim 128, 32768 keys, bf16).

Timing. K steps are timed between two synchronisations (host clock and HIP events on the
launch stream). That bracket is repeated back to back, on a context that keeps growing by
one key per step, until the timed steps add up to a multiple of 64 and to at least 128:
the HashAttention plan hashes new keys 64 at a time (one extra launch pair every 64 steps),
so a multiple of 64 steps holds exactly its share of that work whatever K is. `value` is
the mean over all timed steps; the median and minimum over the K-step brackets are
reported beside it. Before the W warm-up steps bench.py runs untimed steps of its own until
256 steps have run (`clock_settle_steps` in the output): a GPU that had no work for some
milliseconds runs its first ~10 ms of work at a lower clock, and W = 5 with K = 20 would time
nothing else.

Prints ONE JSON line: whole-step microseconds (`value`), the roofline of the dominant kernel
from HIP-event timings taken inside this run, the parity of the last timed step against the
CPU oracle, the oracle timed on the host cores, and short sub-runs of the other headline
configurations (`other_configs`).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "sparse-attention-hub_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0
OUTLIER_CHANNELS = (7, 33, 71, 101)
HASH_BLOCK = 64  # the decode plan hashes new keys this many at a time

WORKLOADS = {
    1: dict(name="cfg1 Sink128+Local256 fp32 B1 Lk4096", B=1, Lk=4096, dtype="f32", sink=128, local=256, kind="none", k=0),
    2: dict(name="cfg2 Sink128+Local512+OracleTopK5% bf16 B4 Lk32768", B=4, Lk=32768, dtype="bf16", sink=128, local=512,
            kind="oracle", k=1638, outliers=True),
    3: dict(name="cfg3 Sink128+Local512+HashAttention top-2048 bf16 B8 Lk32768", B=8, Lk=32768, dtype="bf16", sink=128,
            local=512, kind="hash", k=2048),
    4: dict(name="cfg4 Sink128+Local256+PQCache top-1024 bf16 B4 Lk32768", B=4, Lk=32768, dtype="bf16", sink=128, local=256,
            kind="pq", k=1024, outliers=True),
    5: dict(name="cfg5 Sink128+Local1024+OracleTopK2%+AdaptiveSampling(1%, eps=delta=0.05) bf16 B16 Lk131072", B=16,
            Lk=131072, dtype="bf16", sink=128, local=1024, kind="oracle", k=2621, outliers=True,
            adaptive=dict(rate=0.01, epsilon=0.05, delta=0.05)),
    # the reference's own PQCache example (docs/baselines/pqcache.md:10-27: Sink 128 + Local 128 + PQCache 10 %, two
    # sub-vectors of 64, 6 bits, 10 Lloyd iterations, 32K context, one query); its published 0.867 ms (unnamed CUDA GPU,
    # docs/baselines/pqcache.md:50-61) is context, not a baseline for this hardware
    6: dict(name="ref-docs PQCache: Sink128+Local128+PQCache(10%, group factor 2, 6 bits) bf16 B1 Lk32768", B=1, Lk=32768,
            dtype="bf16", sink=128, local=128, kind="pq", k=3276, outliers=True, pq_group_factor=2, pq_bits=6),
}
HQ, HKV, D = 32, 8, 128
SETTLE_STEPS = 256   # untimed steps before the first bracket, the W warm-up steps included


def algorithmic_bytes(w, sampled_per_row: float = 0.0) -> dict:
    """Unique bytes that must cross HBM once per warm layer-step:
    sink/local rows shared by the 4 query heads of a KV group, top-k rows not shared,
    int32 indices written once and read once, Q and out."""
    es = 4 if w["dtype"] == "f32" else 2
    row = D * es
    B, Lk = w["B"], w["Lk"]
    R = B * HQ
    fixed = w["sink"] + w["local"]
    # `sampled_per_row`: mean number of columns the adaptive sampler added to a row (data dependent, measured)
    gather_topk = int(R * (w["k"] + sampled_per_row) * row * 2)
    gather_fixed = B * HKV * fixed * row * 2
    idx = int(R * (fixed + w["k"] + 2 * sampled_per_row) * 4 * 2)   # sampled entries carry a 4-byte weight too
    qo = 2 * R * D * es
    # one 4-byte signature per (query head, key): the sign plane the decode kernel scans (the non-zero plane of the
    # two-plane cache is read only for the few keys that have a zero component)
    scan = {"none": 0, "oracle": B * HKV * Lk * row, "hash": R * Lk * 4, "pq": B * HKV * (Lk - w["sink"]) * w.get("pq_group_factor", 16)}[w["kind"]]
    attn = gather_topk + gather_fixed + int(R * (fixed + w["k"] + 2 * sampled_per_row) * 4) + qo
    return dict(step=gather_topk + gather_fixed + idx + qo + scan, attention_kernel=attn, scan=scan)


def measured_traffic(kernel: str, cfg: int):
    """(HBM bytes per launch of `kernel`, file) from the committed rocprofv3 PMC summary, if there is one."""
    rel = os.path.join("profiles", f"{kernel}_cfg{cfg}_hbm_traffic.txt")
    try:
        for line in open(os.path.join(ROOT, rel)):
            if line.startswith("hbm_bytes_per_launch"):
                return int(line.split("=")[1]), rel
    except OSError:
        pass
    return None, None


def build_workload(w, device, total_keys, host_rng=True):
    """The chain, 64 query sets and K / V of `total_keys` keys. `host_rng`: N(0, 1) drawn on the host with seed 0
    and cast (the headline run, reproducible everywhere); otherwise drawn on the device (the short sub-runs: config 5
    holds 2 x 2.1 G elements)."""
    import torch

    from sparse_attention_hub_amd.sparse_attention import (
        AdaptiveSamplingMaskerConfig, HashAttentionTopKMaskerConfig, LocalMaskerConfig, OracleTopKConfig, PQCacheConfig, ResearchAttention,
        ResearchAttentionConfig, SinkMaskerConfig,
    )
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    dtype = torch.float32 if w["dtype"] == "f32" else torch.bfloat16
    B = w["B"]
    if host_rng:
        g = torch.Generator().manual_seed(0)
        k = torch.randn(B, HKV, total_keys, D, generator=g)
        v = torch.randn(B, HKV, total_keys, D, generator=g)
        qs = torch.randn(64, B, HQ, 1, D, generator=g)
        if w.get("outliers"):
            for c in OUTLIER_CHANNELS:
                k[..., c] *= 8.0
        k, v, qs = k.to(dtype).to(device), v.to(dtype).to(device), qs.to(dtype).to(device)
    else:
        g = torch.Generator(device=device).manual_seed(0)
        k = torch.randn(B, HKV, total_keys, D, generator=g, device=device, dtype=dtype)
        v = torch.randn(B, HKV, total_keys, D, generator=g, device=device, dtype=dtype)
        qs = torch.randn(64, B, HQ, 1, D, generator=g, device=device, dtype=dtype)
        if w.get("outliers"):
            for c in OUTLIER_CHANNELS:
                k[..., c] *= 8.0
    cfgs = [SinkMaskerConfig(sink_size=w["sink"]), LocalMaskerConfig(window_size=w["local"])]
    extra = {}
    if w["kind"] == "oracle":
        cfgs.append(OracleTopKConfig(heavy_size=w["k"]))
    elif w["kind"] == "hash":
        wts = random_hat_weights(2, HQ, D, 32, 3, 128, dtype=dtype, seed=1)   # layer 1: the second cold call only
        extra["hat_weights"] = wts
        cfgs.append(HashAttentionTopKMaskerConfig(heavy_size=w["k"], hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                                  hat_mlp_activation="silu", hat_weights=wts))
    elif w["kind"] == "pq":
        cfgs.append(PQCacheConfig(heavy_size=w["k"], pq_group_factor=w.get("pq_group_factor", 16), pq_bits=w.get("pq_bits", 8),
                                  kmeans_iter=10, init_offset=w["sink"], metric="euclidean"))
    if w.get("adaptive"):
        a = w["adaptive"]
        cfgs.append(AdaptiveSamplingMaskerConfig(base_rate_sampling=a["rate"], epsilon=a["epsilon"], delta=a["delta"],
                                                 init_offset=w["sink"], local_offset=w["local"]))
    extra["config"] = ResearchAttentionConfig(masker_configs=cfgs)
    ra = ResearchAttention.create_from_config(extra["config"])
    if w.get("adaptive"):
        ra.maskers[-1].seed = 0
    ra.return_attention_weights = False  # HF attention modules drop the dense probabilities in decode
    return ra, qs, k, v, extra


def repeats_for(steps: int) -> int:
    """Number of K-step brackets so that the timed steps are a multiple of 64 and at least 128."""
    reps = HASH_BLOCK // math.gcd(steps, HASH_BLOCK)
    while steps * reps < 2 * HASH_BLOCK:
        reps *= 2
    return reps


def median(xs):
    s = sorted(xs)
    return s[len(s) // 2] if len(s) % 2 else 0.5 * (s[len(s) // 2 - 1] + s[len(s) // 2])


class Run:
    """One workload on the GPU: cold call, warm-up, timed brackets; keeps the last step's output and rows."""

    def __init__(self, w, dev, steps, warm, reps, probe, host_rng, settle=0, hf_layers=0):
        import torch

        self.torch = torch
        self.w, self.dev, self.steps, self.warm, self.reps, self.probe = w, dev, steps, warm, reps, probe
        self.total = steps * reps
        # Steps run before the W warm-up steps so that the clocks have settled when the first bracket starts: after
        # some milliseconds without work the GPU runs its first ~10 ms of work at a lower clock (config 3: 64 us per
        # step falling to 60.5 over the first ~150 steps), which W = 5 warm-up steps and 20-step brackets never leave.
        self.settle = settle
        self.first = w["Lk"] - (settle + warm + self.total)  # the last timed step runs at exactly Lk keys
        if self.first <= w["sink"] + w["local"] + w["k"] + 512:
            raise SystemExit(f"bench.py: {settle} + {warm} + {self.total} steps do not fit below {w['Lk']} keys")
        self.ra, self.qs, self.k, self.v, self.extra = build_workload(w, dev, w["Lk"] + probe, host_rng)
        self.meta = {}
        self.scaling = D ** -0.5
        # hf_layers > 0: every step enters through the callable ModelAdapterHF registers in HuggingFace's attention
        # registry, with what HuggingFace passes it in a decode step of an unpadded batch: the attention module (its
        # layer_idx), the eager mask - a (B, 1, 1, keys) tensor of zeros, a new one per forward pass, i.e. every
        # `hf_layers` layer-steps - and sparse_meta_data among the keyword arguments. (Every timed step here has one
        # key more than the one before, where the layers of one forward pass share a key count: the mask is as wide
        # as the final key count and every step uses its first n_keys columns, as the reference slices it.)
        self.hf_layers = hf_layers
        if hf_layers:
            from types import SimpleNamespace

            from sparse_attention_hub_amd.adapters import ModelAdapterHF

            adapter = ModelAdapterHF(None, self.extra["config"])        # default arguments
            self.ra = adapter.sparse_attention
            self.hf_fn = adapter.get_custom_attention_function(self.ra)
            self.hf_module = SimpleNamespace(layer_idx=0, training=False)
            self.hf_mask = None
            self.hf_calls = 0

    def step(self, i, n_keys, layer=0):
        if self.hf_layers:
            if self.hf_calls % self.hf_layers == 0:
                self.hf_mask = self.torch.zeros((self.w["B"], 1, 1, self.k.shape[2]), dtype=self.qs.dtype, device=self.dev)
            self.hf_calls += 1
            return self.hf_fn(self.hf_module, self.qs[i % self.qs.shape[0]], self.k[:, :, :n_keys], self.v[:, :, :n_keys],
                              self.hf_mask, scaling=self.scaling, dropout=0.0, sparse_meta_data=self.meta)
        return self.ra.custom_attention(None, self.qs[i % self.qs.shape[0]], self.k[:, :, :n_keys], self.v[:, :, :n_keys], None,
                                        self.scaling, 0.0, sparse_meta_data=self.meta, layer_idx=layer)

    def cold(self, second_layer=True):
        """The first call of a layer (it hashes / clusters every key), timed on the host clock with the library's
        per-kernel HIP events on: once for layer 0 - the process's first call, which also loads the code object,
        creates the plan and its buffers - and once more for a second layer index on the same keys, which pays only
        what every further layer of a model pays. Returns the two wall times and the kernel time inside each."""
        from sparse_attention_hub_amd import _native as N

        torch = self.torch
        out = {}
        for name, layer in (("first_call", 0), ("next_layer_cold", 1)):
            if layer and (not second_layer or self.hf_layers):
                break
            torch.cuda.synchronize()
            N.timing_enable(True)
            t0 = time.perf_counter()
            self.step(0, self.first, layer)
            torch.cuda.synchronize()
            out[name + "_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
            kt = N.timing_collect()
            N.timing_enable(False)
            out[name + "_kernels_ms"] = round(sum(ms for _, ms in kt.values()), 2)
        for per_layer in self.meta.values():       # the second layer's caches are not needed again
            if isinstance(per_layer, dict):
                per_layer.pop(1, None)
        return out

    def timed(self):
        """(wall ms per bracket, HIP-event ms per bracket, host launch-loop ms per bracket, HIP-event ms per step over
        each bracket's steps after the first few: by then the host runs ahead of the GPU, so that region holds kernels
        back to back without the start-up gap of a bracket that begins on an idle GPU)."""
        torch = self.torch
        for i in range(self.settle + self.warm):
            self.step(i, self.first + 1 + i)
        torch.cuda.synchronize()
        wall, gpu, host, inner = [], [], [], []
        n = self.first + self.settle + self.warm
        skip = min(4, self.steps // 2)
        for _ in range(self.reps):
            ev0, ev1, evm = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ev0.record()
            for i in range(self.steps):
                if i == skip:
                    evm.record()
                n += 1
                self.last_q = i % self.qs.shape[0]
                self.last_out, _ = self.step(i, n)
            ev1.record()
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            wall.append((t2 - t0) * 1e3)
            host.append((t1 - t0) * 1e3)
            gpu.append(ev0.elapsed_time(ev1))
            inner.append(evm.elapsed_time(ev1) / (self.steps - skip))
        assert n == self.w["Lk"]
        self.last = self.last_state()
        return wall, gpu, host, inner

    def last_state(self):
        """What the parity check needs of the last timed step: output, query set, selected columns, warm-cache extent."""
        rows = self.last_rows()
        cache = self.meta.get("key", {}).get(0) if self.w["kind"] == "hash" else None
        last = dict(out=self.last_out, q=self.last_q, n_hashed=getattr(cache, "n", 0),
                    cols=None if rows is None else rows[0].clone(), cnt=None if rows is None else rows[1].clone())
        if self.w.get("adaptive"):
            masker = self.ra.maskers[-1]
            last["budget"] = masker.last_budget.clone()
            last["adaptive_call"] = masker.call_index - 1
        return last

    def last_rows(self):
        """(cols int32 [R, cap], cnt int32 [R]) of the last step's mask, or None when no row list was written."""
        if self.w.get("adaptive"):
            rows = self.ra.maskers[-1].last_rows
            return rows.cols, rows.cnt
        plan = next(iter(self.ra._plans.values()), None)
        if plan is None or plan.cols is None or self.w["kind"] == "none":
            return None
        return plan.cols, plan.cnt

    def instrumented(self):
        """Per-kernel durations: HIP events around every launch, `probe` more steps on the same buffers."""
        from sparse_attention_hub_amd import _native as N

        N.timing_enable(True)
        for i in range(self.probe):
            self.step(i, self.w["Lk"] + 1 + i)
        self.torch.cuda.synchronize()
        kt = N.timing_collect()
        N.timing_enable(False)
        return {name: dict(launches=c, avg_us=1e3 * ms / c) for name, (c, ms) in kt.items()}


def oracle_specs(run, n_keys, n_hashed, b=0, adaptive_call=0):
    """Masker specs and warm state (batch row `b`) for `oracle.reference_path.research_attention`."""
    w, extra, meta = run.w, run.extra, run.meta
    specs = [("sink", w["sink"]), ("local", w["local"])]
    state = {}
    if w["kind"] == "oracle":
        specs.append(("oracle_topk", w["k"]))
    elif w["kind"] == "hash":
        specs.append(("hash_topk", w["k"], extra["hat_weights"][0], "silu"))
        cache = meta["key"][0]
        sub = type(cache).__new__(type(cache))            # one batch row, the keys hashed when the step ran
        sub.bits, sub.n, sub.codes = cache.bits, n_hashed, cache.codes[b:b + 1]
        state["key_sig"] = sub.unpack(run.qs.dtype).cpu()
    elif w["kind"] == "pq":
        cent = meta["pq_centroids"][0][b:b + 1].cpu()
        book = meta["pq_codebook"][0].to_reference()[b:b + 1, : n_keys - w["sink"]].cpu()
        if book.shape[1] < n_keys - w["sink"]:
            # keys not quantised yet sit inside the local window (the plan quantises them a block at a time): the
            # oracle scores every key beyond init_offset, so they get a stand-in code; they are active already
            pad = book[:, -1:].expand(-1, n_keys - w["sink"] - book.shape[1], -1, -1)
            book = __import__("torch").cat([book, pad], dim=1)
        specs.append(("pq_topk", w["k"], w["sink"], cent, book))
    if w.get("adaptive"):
        a = w["adaptive"]
        # the Philox stream of the masker's call (seed 0, offset 2 x its index)
        specs.append(("adaptive", a["rate"], a["epsilon"], a["delta"], w["sink"], w["local"], 0, 2 * adaptive_call))
    return specs, state


def parity_and_cpu_baseline(run, last, budget_s=25.0):
    """The reference algorithm (dense masks, repeat_kv, full-key fp32 softmax) as restated by the oracle, on single
    batch rows of the last timed step: first as the checker of that step's output and selected columns (batch rows 0
    and B - 1; the adaptive chain: row 0, whose mask rows carry the Philox row indices the oracle uses), then timed on
    the host cores on row 0 and scaled by the batch size (batch rows are independent). Warm caches (key signatures / PQ
    codes) are the GPU run's, so only the layer-step is restated."""
    import torch

    from oracle import reference_path as O

    w = run.w
    B = w["B"]
    n_keys = w["Lk"]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    adaptive = bool(w.get("adaptive"))
    tol = 1e-5 if w["dtype"] == "f32" else 2e-2

    def inputs(b):
        q = run.qs[last["q"]][b:b + 1].cpu()
        k = run.k[b:b + 1, :, :n_keys].cpu()
        v = run.v[b:b + 1, :, :n_keys].cpu()
        specs, state = oracle_specs(run, n_keys, last["n_hashed"], b, last.get("adaptive_call", 0))
        if w["kind"] == "hash":
            # the query's signature bits as the kernels compute them (a float MLP on the host may round a borderline
            # output to the other side of zero)
            qcodes = torch.empty((HQ, 2), dtype=torch.int32, device=run.dev)
            run.ra.maskers[2]._hash(run.qs[last["q"]][b:b + 1], HQ, HQ, 0, 1, 0, "query", qcodes, 1, 0)
            c = qcodes.cpu().to(torch.int64) & 0xFFFFFFFF
            shifts = torch.arange(32)
            state["query_sig"] = ((((c[:, 0:1] >> shifts) & 1) * 2 - 1) * ((c[:, 1:2] >> shifts) & 1)).to(q.dtype).view(1, HQ, 1, 32)
        if adaptive:
            state["budget"] = last["budget"][b * HQ:(b + 1) * HQ].long().cpu()     # the kernels' budgets: sets given the budget
        return q, k, v, specs, state

    def membership(b):
        cols = last["cols"][b * HQ:(b + 1) * HQ].long().cpu()
        cnt = last["cnt"][b * HQ:(b + 1) * HQ].long().cpu()
        member = torch.zeros((HQ, n_keys), dtype=torch.bool)
        for r in range(HQ):
            member[r, cols[r, : cnt[r]]] = True
        return member

    rows_checked = [0] if adaptive or B == 1 else [0, B - 1]
    worst_err, sets_equal, overlap = 0.0, True, 1.0
    times = []
    for b in rows_checked:
        q, k, v, specs, state = inputs(b)
        t0 = time.perf_counter()
        oo, _, om = O.research_attention(specs, q, k, v, None, D ** -0.5, state=dict(state))
        if b == 0:
            times.append(time.perf_counter() - t0)
        got = last["out"][b:b + 1].float().cpu()
        worst_err = max(worst_err, ((got - oo.float()).norm() / oo.float().norm()).item())
        if last["cols"] is not None:
            want = om.to_dense()[0, :, 0] != 0
            member = membership(b)
            sets_equal = sets_equal and bool(torch.equal(member, want))
            overlap = min(overlap, float((member & want).sum()) / float(want.sum()))
    parity = dict(rel_err=float(f"{worst_err:.3e}"), tolerance=tol,
                  rows_checked=f"batch rows {rows_checked} ({HQ} mask rows each, of {B * HQ}) of the last timed step; worst row reported")
    if last["cols"] is not None:
        parity["index_sets_equal"] = sets_equal
        parity["index_set_overlap"] = round(overlap, 6)
    if adaptive:
        parity["note"] = ("sampled sets compared given the kernels' budgets (the budget itself is a float formula truncated to an "
                          "integer, compared with the oracle's to one unit of precision in the tests)")
        b_or = None
        q, k, v, specs, state = inputs(0)
        st = {kk: vv for kk, vv in state.items() if kk != "budget"}
        O.research_attention(specs, q, k, v, None, D ** -0.5, state=st)
        b_or = st["budget_oracle"].reshape(-1).double()
        b_k = state["budget"].double()
        parity["budget_max_rel_diff_vs_oracle"] = float(f"{((b_k - b_or).abs() / b_or.clamp_min(1)).max().item():.3e}")
    # CPU baseline: more timed passes over batch row 0 within the budget
    q, k, v, specs, state = inputs(0)
    t_all = time.perf_counter()
    while len(times) < 12 and (len(times) < 2 or time.perf_counter() - t_all < budget_s):
        t0 = time.perf_counter()
        O.research_attention(specs, q, k, v, None, D ** -0.5, state=dict(state))
        times.append(time.perf_counter() - t0)
    per_row = median(times[1:] or times)
    base = dict(value=round(per_row * B * 1e6, 1), unit="us/layer-step", cores=cores, kind="port",
                sample=f"oracle (torch-CPU restatement of the reference path) on 1 of {B} batch rows, "
                       f"median of {max(1, len(times) - 1)} warm steps x {B}; torch threads={cores}")
    return parity, base


def hf_callable_run(w, dev, steps, warm, reps, probe, settle, direct_us, direct_out, layers=32) -> dict:
    """The same workload and the same timed brackets, entered the way HuggingFace enters: through the callable
    `ModelAdapterHF` (default arguments) registers, with the attention module, the eager mask of an unpadded decode
    step (zeros, a new tensor every `layers` layer-steps = once per forward pass of a `layers`-layer model) and
    sparse_meta_data as a keyword argument."""
    import torch

    run = Run(w, dev, steps, warm, reps, probe, host_rng=True, settle=settle, hf_layers=layers)  # same seeded inputs
    run.cold(second_layer=False)
    wall, gpu, host, _ = run.timed()
    total = run.total
    per_bracket_us = [x / steps * 1e3 for x in wall]
    us = sum(wall) / total * 1e3
    same = bool(torch.equal(run.last_out, direct_out))
    return dict(us=round(us, 2), median_us=round(median(per_bracket_us), 2), min_us=round(min(per_bracket_us), 2),
                gpu_us=round(sum(gpu) / total * 1e3, 2), host_launch_us=round(sum(host) / total * 1e3, 2),
                delta_vs_value_us=round(us - direct_us, 2), timed_steps_total=total, forward_pass_layers=layers,
                last_output_bit_identical_to_direct_call=same,
                entry="callable of ModelAdapterHF.get_custom_attention_function (default adapter arguments): module with "
                      "layer_idx, additive mask = zeros of shape (B, 1, 1, keys) in the query dtype re-created once per "
                      f"{layers} layer-steps, sparse_meta_data in kwargs; the mask is classified on the device once per "
                      "tensor (one launch and one read-back), then every layer-step of that pass is the one-kernel plan")


def sub_run(cfg: int, dev, cpu_budget_s: float) -> dict:
    """A run of another configuration of the headline set: the two cold calls, warm-up steps (about 10 ms of them, so
    that the clocks have settled), two brackets of 64 timed steps, parity of the last step against the oracle and the
    oracle timed on the host cores (bounded by `cpu_budget_s`)."""
    import torch

    w = dict(WORKLOADS[cfg])
    steps, reps = 64, 2
    run = Run(w, dev, steps, 8 if cfg == 5 else 160, reps, 0, host_rng=False)
    cold = run.cold()
    wall, gpu, _, _ = run.timed()
    total = steps * reps
    sampled = 0.0
    if w.get("adaptive"):
        sampled = float(run.ra.maskers[-1].last_rows.cnt.float().mean().item()) - (w["sink"] + w["local"] + w["k"])
    ab = algorithmic_bytes(w, sampled)["step"]
    per_bracket_us = [x / steps * 1e3 for x in wall]
    us, gpu_us = sum(wall) / total * 1e3, sum(gpu) / total * 1e3
    out = dict(workload=w["name"], us=round(us, 2), median_us=round(median(per_bracket_us), 2), min_us=round(min(per_bracket_us), 2),
               gpu_us=round(gpu_us, 2), timed_steps_total=total, brackets=reps, algorithmic_bytes=ab,
               achieved_GBps=round(ab / (gpu_us * 1e-6) / 1e9, 1), frac=round(ab / (gpu_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
               data="synthetic, drawn on the device", **cold)
    if w.get("adaptive"):
        out["keys_per_row"] = round(w["sink"] + w["local"] + w["k"] + sampled, 1)
    if cpu_budget_s > 0:
        out["parity"], out["cpu_baseline"] = parity_and_cpu_baseline(run, run.last, cpu_budget_s)
    del run
    torch.cuda.empty_cache()
    return out


def cold_probe(dev) -> dict:
    """The matrix-core kernels of the cold calls at the shapes of the headline configurations, timed with HIP events: two Lloyd iterations
    of the config-4 k-means (4 x 8 KV heads x 16 sub-spaces, 32640 keys, 256 centres, sub-vectors of 8) and the
    config-3 bulk signature build (8 x 32 heads x 32768 keys, MLP 128-128-128-32)."""
    import torch

    from sparse_attention_hub_amd.sparse_attention import HashAttentionTopKMasker, HashAttentionTopKMaskerConfig
    from sparse_attention_hub_amd.sparse_attention.research_attention.maskers.fixed.implementations.utils.pq_utils import kmeans_keys_batched
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    dtype = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    k4 = torch.randn(4, HKV, 32768, D, generator=g, device=dev, dtype=dtype)
    for c in OUTLIER_CHANNELS:
        k4[..., c] *= 8.0
    codes = torch.zeros((4, HKV, 32768 - 128, 16), dtype=torch.uint8, device=dev)
    from sparse_attention_hub_amd import _native as N

    kmeans_keys_batched(k4, 128, 16, 256, 1, codes, 32768 - 128, seed=0)       # warm-up (module load)
    k3 = torch.randn(8, HKV, 32768, D, generator=g, device=dev, dtype=dtype)
    wts = random_hat_weights(1, HQ, D, 32, 3, 128, dtype=dtype, seed=1)
    m = HashAttentionTopKMasker(HashAttentionTopKMaskerConfig(heavy_size=2048, hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                                             hat_mlp_activation="silu", hat_weights=wts))
    m._update_key_signatures(k3[:, :, :4096], HQ, {}, 0)                       # warm-up
    torch.cuda.synchronize()
    N.timing_enable(True)                                                      # HIP events around every launch of the library
    kmeans_keys_batched(k4, 128, 16, 256, 2, codes, 32768 - 128, seed=0)
    m._update_key_signatures(k3, HQ, {}, 0)
    torch.cuda.synchronize()
    kt = N.timing_collect()
    N.timing_enable(False)
    lloyd_ms = kt["k_pq_assign_mfma"][1] / kt["k_pq_assign_mfma"][0]
    sig_ms = kt["k_hash_sig_mfma"][1] / kt["k_hash_sig_mfma"][0]
    lloyd_flop = 2.0 * 4 * HKV * 16 * (32768 - 128) * 256 * 8
    sig_flop = 2.0 * 8 * HQ * 32768 * (128 * 128 + 128 * 128 + 128 * 32)
    return {"cold_probe": True,
            "k_pq_assign_mfma_ms": round(lloyd_ms, 3), "k_pq_assign_mfma_TFLOPs": round(lloyd_flop / lloyd_ms / 1e9, 1),
            "k_pq_assign_mfma_frac_of_fp32_mfma_peak": round(lloyd_flop / lloyd_ms / 1e9 / 157.3, 4),
            "k_hash_sig_mfma_ms": round(sig_ms, 3), "k_hash_sig_mfma_TFLOPs": round(sig_flop / sig_ms / 1e9, 1),
            "k_hash_sig_mfma_frac_of_bf16_mfma_peak": round(sig_flop / sig_ms / 1e9 / 2500.0, 4),
            "kernels_avg_ms": {n: round(ms / c, 4) for n, (c, ms) in sorted(kt.items())},
            "note": "HIP events around every launch; flops = 2 x keys x centres x dims (k-means), 2 x MLP multiply-adds (signatures)"}


def hw_probe(dev) -> dict:
    """What the GPU gives to two patterns of the library (the bench-only object `bench_hw_probe.so`, built from
    `bench_hw_probe.hip` beside this file; HIP events around back-to-back launches): a 4 GiB read stream alone and with
    1/32 of its volume written back (the exact-score pass over K at config 5), and matrix / vector / interleaved
    instruction streams (the Lloyd assignment)."""
    import ctypes

    import torch

    from sparse_attention_hub_amd import _native as N

    path = os.path.join(ROOT, "bench_hw_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} not found: `python __graft_entry__.py` builds it")
    probe = ctypes.CDLL(path).bench_hw_probe
    probe.restype = ctypes.c_int
    probe.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                      ctypes.c_int, ctypes.c_void_p]

    out = {"hw_probe": True}
    n = 4 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty(n // 32 + 4096, dtype=torch.uint8, device=dev)
    stream = N.stream_ptr(dev)

    def timed(args, reps):
        for _ in range(3):
            if probe(*args) != 0:
                raise RuntimeError(f"bench_hw_probe refused {args}")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            probe(*args)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    names = {0: "read_4GiB", 1: "read_4GiB_write_4x128B_per_16KB", 2: "read_4GiB_write_512B_per_16KB"}
    for kind in (0, 1, 2, 0):
        us = timed((kind, src.data_ptr(), n, dst.data_ptr(), dst.numel(), 0, 0, stream), 10)
        out.setdefault(names[kind], []).append({"us": round(us, 1), "read_TBps": round(n / us / 1e6, 3)})
    names = {3: "matrix_only", 4: "vector_only", 5: "matrix_and_vector_interleaved"}
    for wgs in (256, 1024):
        for kind in (3, 4, 5):
            us = timed((kind, None, 0, dst.data_ptr(), dst.numel(), 2000, wgs, stream), 5)
            out[f"{names[kind]}_{wgs // 256}_waves_per_simd_us"] = round(us, 1)
    out["note"] = ("stream kinds: 65536 workgroups x 64 KB, non-temporal 16-byte loads; issue kinds: 2000 iterations of 4 dependent "
                   "32x32x2 fp32 matrix instructions and / or 48 vector FMAs per wave")
    return out


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=20,
                    help="untimed steps before the first bracket (bench.py runs untimed steps of its own before them "
                         "until SETTLE_STEPS have run, so that the clocks have settled)")
    ap.add_argument("--config", type=int, default=3, choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-hf-callable", action="store_true", help="skip the sub-run that enters through the HuggingFace callable")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the short sub-runs of the other configurations")
    ap.add_argument("--batch", type=int, default=0, help="study only: override the workload's batch size")
    ap.add_argument("--keys", type=int, default=0, help="study only: override the workload's key count")
    ap.add_argument("--cold-probe", action="store_true",
                    help="short run for `rocprofv3 --pmc` / `--kernel-trace` of the two matrix-core kernels of the cold calls: "
                         "two Lloyd iterations of the config-4 k-means and the config-3 bulk signature build")
    ap.add_argument("--hw-probe", action="store_true",
                    help="times the probe kernels of bench_hw_probe.so: read-stream ceilings with and without a write stream, "
                         "matrix / vector instruction overlap")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="short run for `rocprofv3 --pmc`: a few layer-steps plus three 256 MiB copy kernels of known size")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on ONE GPU (no collectives on the decode path); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from sparse_attention_hub_amd import _native as N

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the MI355X kernels have no CPU fallback", file=sys.stderr)
        sys.exit(3)
    N.lib()
    dev = torch.device("cuda:0")
    if args.cold_probe:
        print(json.dumps(cold_probe(dev)))
        return
    if args.hw_probe:
        print(json.dumps(hw_probe(dev)))
        return
    w = dict(WORKLOADS[args.config])
    study = bool(args.batch or args.keys)
    if study:
        w["B"] = args.batch or w["B"]
        w["Lk"] = args.keys or w["Lk"]
        w["name"] += f" [size override: B={w['B']} Lk={w['Lk']}]"
    steps, warm = args.steps, args.warmup
    reps = repeats_for(steps)
    probe = 2 * HASH_BLOCK                                # instrumented steps for the per-kernel durations
    settle = max(0, SETTLE_STEPS - warm)
    run = Run(w, dev, steps, warm, reps, probe, host_rng=True, settle=settle)
    cold = run.cold()

    if args.pmc_probe:
        for i in range(5):
            run.step(i, run.first + 1 + i)
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)                                # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        print(json.dumps({"pmc_probe": True, "copy_bytes": src.numel(), "steps": 5}))
        return

    wall, gpu, host, inner = run.timed()
    total = run.total
    ms_per_step = sum(wall) / total
    gpu_ms_per_step = sum(gpu) / total
    last = run.last

    kernels = run.instrumented()
    sampled = 0.0
    if w.get("adaptive"):
        # mean entries per row after the last step, minus what the fixed maskers put there
        sampled = float(run.ra.maskers[-1].last_rows.cnt.float().mean().item()) - (w["sink"] + w["local"] + w["k"])
    ab = algorithmic_bytes(w, sampled)
    periodic = {n: d for n, d in kernels.items() if n in ("k_hash_sig_small_mfma", "k_hash_sig_gemv", "k_hash_compact")}
    amortised_hash_us = sum(d["avg_us"] * d["launches"] for d in periodic.values()) / probe
    # the dominant kernel: the attention kernel, or - when selection and attention of a step run as one
    # kernel - that kernel, whose algorithmic bytes are then the whole step's
    if "k_hash_decode_attn" in kernels:
        # One launch per step: an event pair around back-to-back steps times their launches without the gaps an event
        # pair around every single launch adds. The periodic hashing launches (one pair every 64 steps) that fall
        # into the region stay inside this figure: it errs on the long side.
        dom, dom_bytes = "k_hash_decode_attn", ab["step"]
        dom_us = sum(inner) / len(inner) * 1e3
        timing = ("HIP events around the steps of each bracket of K back-to-back steps after its first min(4, K/2) (the kernels "
                  "then run back to back; a bracket starts on an idle GPU and its first launch waits for the host), divided by "
                  "their number, mean over all brackets; one launch per step, the periodic new-key hashing launches included")
        del kernels[dom]                                  # per-launch event pairs measure launch gaps for this one
    elif "k_select16_attn" in kernels:
        # selection and attention of a row in one kernel: the attention's bytes plus the row's 2-byte score keys, read once
        dom, dom_bytes = "k_select16_attn", ab["attention_kernel"] + w["B"] * HQ * w["Lk"] * 2
        dom_us = kernels[dom]["avg_us"]
        timing = "HIP events around every launch"
    else:
        dom, dom_bytes = "k_sparse_attn", ab["attention_kernel"]
        dom_us = kernels[dom]["avg_us"]
        timing = "HIP events around every launch"
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9
    traffic, traffic_file = measured_traffic(dom, args.config)
    roofline = dict(bound="hbm", kernel=dom, achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4), traffic=None if study else traffic,
                    traffic_source=None if study or traffic is None else f"{traffic_file} (rocprofv3 --pmc run of this workload, committed; not re-measured here)",
                    algorithmic_bytes_per_launch=dom_bytes, avg_launch_us=round(dom_us, 2), timing=timing)
    step_gbs = ab["step"] / (ms_per_step * 1e-3) / 1e9
    per_bracket_us = [x / steps * 1e3 for x in wall]
    per_bracket_gpu_us = [x / steps * 1e3 for x in gpu]

    out = {
        "metric": "sparse decode \u00b5s/layer-step at 32K/128K ctx; achieved HBM GB/s vs peak",
        "value": round(ms_per_step * 1e3, 2),
        "unit": "us/layer-step",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warm,
        "clock_settle_steps": settle,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w["dtype"],
        "data": "synthetic",
        "config": {"workload": w["name"], "q_heads": HQ, "kv_heads": HKV, "head_dim": D, "batch": w["B"], "keys": w["Lk"],
                   "keys_per_row": round(w["sink"] + w["local"] + w["k"] + sampled, 1), "attention_weights_output": False},
        "timed_steps_total": total,
        "brackets": reps,
        "median_us": round(median(per_bracket_us), 2),
        "min_us": round(min(per_bracket_us), 2),
        "gpu_ms_per_step": round(gpu_ms_per_step, 5),
        "gpu_median_us": round(median(per_bracket_gpu_us), 2),
        "gpu_min_us": round(min(per_bracket_gpu_us), 2),
        "host_launch_ms_per_step": round(sum(host) / total, 5),
        "step_algorithmic_bytes": ab["step"],
        "step_achieved_GBps": round(step_gbs, 1),
        "step_frac_of_hbm_peak": round(step_gbs / HBM_PEAK_GBS, 4),
        **cold,
        "amortised_hash_us": round(amortised_hash_us, 3),
        "kernels_avg_us": {n: round(d["avg_us"], 2) for n, d in sorted(kernels.items())},
        "kernels_avg_us_note": "HIP events around every single launch (they include the event markers' own gaps)",
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["parity"], out["cpu_baseline"] = parity_and_cpu_baseline(run, last)
    if not study and not args.no_hf_callable:
        del run
        torch.cuda.empty_cache()
        out["hf_callable"] = hf_callable_run(w, dev, steps, warm, reps, probe, settle, out["value"], last["out"])
        run = None
    if not args.no_other_configs and not study:
        del last
        run = None
        torch.cuda.empty_cache()
        others = {}
        for cfg in sorted(WORKLOADS):
            if cfg != args.config:
                others[f"cfg{cfg}"] = sub_run(cfg, dev, 0.0 if args.no_cpu_baseline else 4.0)
        out["other_configs"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
