#!/usr/bin/env python3
"""Decode layer-step benchmark of the MI355X ResearchAttention path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1|2|3|4]

A step is one `ResearchAttention.custom_attention` call with one query token on a warm
cache (hash signatures / PQ codes of all earlier keys already built, one new key appended
per step), on synthetic inputs that are resident in HBM before the timed region. Default
workload: BASELINE config 3, the one the headline target is quoted on (Sink 128 + Local 512
+ HashAttention top-2048, batch 8, 32 query / 8 KV heads, head_dim 128, 32768 keys, bf16).

Prints ONE JSON line: whole-step microseconds (`value`), the roofline of the dominant kernel
from HIP-event timings taken inside this run, and the CPU oracle timed on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "sparse-attention-hub_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0
OUTLIER_CHANNELS = (7, 33, 71, 101)

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
}
HQ, HKV, D = 32, 8, 128


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
    scan = {"none": 0, "oracle": B * HKV * Lk * row, "hash": R * Lk * 4, "pq": B * HKV * (Lk - w["sink"]) * 16}[w["kind"]]
    attn = gather_topk + gather_fixed + int(R * (fixed + w["k"] + 2 * sampled_per_row) * 4) + qo
    return dict(step=gather_topk + gather_fixed + idx + qo + scan, attention_kernel=attn, scan=scan)


def measured_traffic(kernel: str, cfg: int):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 PMC summary, if there is one."""
    path = os.path.join(ROOT, "profiles", f"{kernel}_cfg{cfg}_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.startswith("hbm_bytes_per_launch"):
                return int(line.split("=")[1])
    except OSError:
        pass
    return None


def build_workload(w, device, total_keys):
    import torch

    from sparse_attention_hub_amd.sparse_attention import (
        AdaptiveSamplingMaskerConfig, HashAttentionTopKMaskerConfig, LocalMaskerConfig, OracleTopKConfig, PQCacheConfig, ResearchAttention,
        ResearchAttentionConfig, SinkMaskerConfig,
    )
    from sparse_attention_hub_amd.sparse_attention.utils.hashattention_utils import random_hat_weights

    dtype = torch.float32 if w["dtype"] == "f32" else torch.bfloat16
    g = torch.Generator().manual_seed(0)
    B = w["B"]
    k = torch.randn(B, HKV, total_keys, D, generator=g)
    v = torch.randn(B, HKV, total_keys, D, generator=g)
    if w.get("outliers"):
        for c in OUTLIER_CHANNELS:
            k[..., c] *= 8.0
    qs = torch.randn(64, B, HQ, 1, D, generator=g)
    cfgs = [SinkMaskerConfig(sink_size=w["sink"]), LocalMaskerConfig(window_size=w["local"])]
    extra = {}
    if w["kind"] == "oracle":
        cfgs.append(OracleTopKConfig(heavy_size=w["k"]))
    elif w["kind"] == "hash":
        wts = random_hat_weights(1, HQ, D, 32, 3, 128, dtype=dtype, seed=1)
        extra["hat_weights"] = wts
        cfgs.append(HashAttentionTopKMaskerConfig(heavy_size=w["k"], hat_bits=32, hat_mlp_layers=3, hat_mlp_hidden_size=128,
                                                  hat_mlp_activation="silu", hat_weights=wts))
    elif w["kind"] == "pq":
        cfgs.append(PQCacheConfig(heavy_size=w["k"], pq_group_factor=16, pq_bits=8, kmeans_iter=10, init_offset=w["sink"],
                                  metric="euclidean"))
    if w.get("adaptive"):
        a = w["adaptive"]
        cfgs.append(AdaptiveSamplingMaskerConfig(base_rate_sampling=a["rate"], epsilon=a["epsilon"], delta=a["delta"],
                                                 init_offset=w["sink"], local_offset=w["local"]))
    ra = ResearchAttention.create_from_config(ResearchAttentionConfig(masker_configs=cfgs))
    if w.get("adaptive"):
        ra.maskers[-1].seed = 0
    ra.return_attention_weights = False  # HF attention modules drop the dense probabilities in decode
    return ra, qs.to(dtype).to(device), k.to(dtype).to(device), v.to(dtype).to(device), extra


def cpu_baseline(w, extra, ra_meta, k_dev, v_dev, q_dev, n_keys, budget_s=25.0):
    """The reference algorithm (dense masks, repeat_kv, full-key fp32 softmax) as restated by the
    oracle, timed on the host cores for ONE batch row and scaled by the batch size (rows are
    independent); the warm caches are taken from the GPU run so only the layer-step is timed."""
    import torch

    from oracle import reference_path as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    q = q_dev[:1].cpu()
    k = k_dev[:1, :, :n_keys].cpu()
    v = v_dev[:1, :, :n_keys].cpu()
    specs = [("sink", w["sink"]), ("local", w["local"])]
    state = {}
    if w["kind"] == "oracle":
        specs.append(("oracle_topk", w["k"]))
    elif w["kind"] == "hash":
        specs.append(("hash_topk", w["k"], extra["hat_weights"][0], "silu"))
        cache = ra_meta["key"][0]
        sub = type(cache).__new__(type(cache))            # one batch row, the n_keys - 1 earlier keys
        sub.bits, sub.n, sub.codes = cache.bits, n_keys - 1, cache.codes[:1]
        state["key_sig"] = sub.unpack(q.dtype).cpu()
    elif w["kind"] == "pq":
        cent = ra_meta["pq_centroids"][0][:1].cpu()
        book = ra_meta["pq_codebook"][0].to_reference()[:1, : n_keys - w["sink"]].cpu()
        specs.append(("pq_topk", w["k"], w["sink"], cent, book))
    if w.get("adaptive"):
        a = w["adaptive"]
        specs.append(("adaptive", a["rate"], a["epsilon"], a["delta"], w["sink"], w["local"], 0, 0))
    times = []
    t_all = time.perf_counter()
    for it in range(12):
        st = dict(state)
        t0 = time.perf_counter()
        O.research_attention(specs, q, k, v, None, D ** -0.5, state=st)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_all > budget_s and it >= 1:
            break
    per_row = sorted(times[1:] or times)[len(times[1:] or times) // 2]
    return dict(value=per_row * w["B"] * 1e6, unit="us/layer-step", cores=cores, kind="port",
                sample=f"oracle (torch-CPU restatement of the reference path) on 1 of {w['B']} batch rows, "
                       f"median of {max(1, len(times) - 1)} warm steps x {w['B']}; torch threads={cores}")


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=3, choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--batch", type=int, default=0, help="study only: override the workload's batch size")
    ap.add_argument("--keys", type=int, default=0, help="study only: override the workload's key count")
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
    w = dict(WORKLOADS[args.config])
    if args.batch or args.keys:
        w["B"] = args.batch or w["B"]
        w["Lk"] = args.keys or w["Lk"]
        w["name"] += f" [size override: B={w['B']} Lk={w['Lk']}]"
    steps, warm = args.steps, args.warmup
    probe = max(20, min(steps, 100))                      # instrumented steps for the per-kernel roofline
    total_keys = w["Lk"] + probe
    first = w["Lk"] - (warm + steps)                      # the last timed step runs at exactly Lk keys
    ra, qs, k, v, extra = build_workload(w, dev, total_keys)
    meta = {}
    scaling = D ** -0.5

    def step(i, n_keys):
        return ra.custom_attention(None, qs[i % qs.shape[0]], k[:, :, :n_keys], v[:, :, :n_keys], None, scaling, 0.0,
                                   sparse_meta_data=meta, layer_idx=0)

    # cold call: builds all signatures / runs k-means; reported apart
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    step(0, first)
    torch.cuda.synchronize()
    cold_ms = (time.perf_counter() - t0) * 1e3

    if args.pmc_probe:
        for i in range(5):
            step(i, first + 1 + i)
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)                                # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        print(json.dumps({"pmc_probe": True, "copy_bytes": src.numel(), "steps": 5}))
        return

    for i in range(warm):
        step(i, first + 1 + i)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(steps):
        step(i, first + warm + 1 + i)
    ev1.record()
    host_ms = (time.perf_counter() - t0) * 1e3          # launch loop only: host cost when the GPU keeps up
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = ev0.elapsed_time(ev1)
    ms_per_step = wall_ms / steps

    # per-kernel durations, HIP events on the launch stream, same process, same buffers
    N.timing_enable(True)
    for i in range(probe):
        step(i, w["Lk"] + 1 + i)
    torch.cuda.synchronize()
    kt = N.timing_collect()
    N.timing_enable(False)
    kernels = {name: dict(launches=c, avg_us=1e3 * ms / c) for name, (c, ms) in kt.items()}
    sampled = 0.0
    if w.get("adaptive"):
        # mean entries per row after the last step, minus what the fixed maskers put there
        sampled = float(ra.maskers[-1].last_rows.cnt.float().mean().item()) - (w["sink"] + w["local"] + w["k"])
    ab = algorithmic_bytes(w, sampled)
    # the dominant kernel: the attention kernel, or - when selection and attention of a step run as one
    # kernel - that kernel, whose algorithmic bytes are then the whole step's
    if "k_hash_decode_attn" in kernels:
        dom, dom_bytes = "k_hash_decode_attn", ab["step"]
    else:
        dom, dom_bytes = "k_sparse_attn", ab["attention_kernel"]
    dom_us = kernels[dom]["avg_us"]
    timing = "HIP events around every launch"
    if dom == "k_hash_decode_attn":
        # One launch per step: the event pair around the K back-to-back steps of the timed region times K launches
        # without the launch gaps an event pair around each single launch adds. The rare hashing launches of the
        # region (one pair every 64 steps) stay inside this figure, which therefore errs on the long side.
        dom_us = gpu_ms * 1e3 / steps
        timing = "HIP events around the timed region / steps (one launch per step)"
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9
    roofline = dict(bound="hbm", kernel=dom, achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4), traffic=measured_traffic(dom, args.config),
                    algorithmic_bytes_per_launch=dom_bytes, avg_launch_us=round(dom_us, 2), timing=timing)
    step_gbs = ab["step"] / (ms_per_step * 1e-3) / 1e9

    out = {
        "metric": "sparse decode us/layer-step at 32K ctx; achieved HBM GB/s vs peak",
        "value": round(ms_per_step * 1e3, 2),
        "unit": "us/layer-step",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warm,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w["dtype"],
        "data": "synthetic",
        "config": {"workload": w["name"], "q_heads": HQ, "kv_heads": HKV, "head_dim": D, "batch": w["B"], "keys": w["Lk"],
                   "keys_per_row": round(w["sink"] + w["local"] + w["k"] + sampled, 1), "attention_weights_output": False},
        "gpu_ms_per_step": round(gpu_ms / steps, 5),
        "host_launch_ms_per_step": round(host_ms / steps, 5),
        "step_algorithmic_bytes": ab["step"],
        "step_achieved_GBps": round(step_gbs, 1),
        "step_frac_of_hbm_peak": round(step_gbs / HBM_PEAK_GBS, 4),
        "cold_call_ms": round(cold_ms, 2),
        "kernels_avg_us": {n: round(d["avg_us"], 2) for n, d in sorted(kernels.items())},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, extra, meta, k, v, qs[0], w["Lk"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
