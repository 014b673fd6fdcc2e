#!/usr/bin/env python3
"""Throughput of the cascade attention hot path on one MI355X.

A "step" is one pass of the path over one batch of synthetic input: the attention of one
2048-token chunk per stream over [64 sinks | 8 cascades x 2048 slots | chunk] plus the cascading
cache update, on a Llama-3.1-8B-shaped attention layer (32 query / 8 kv heads, head_dim 128,
bf16, 2 streams) whose cache is already full (steady state of the 65536-token stream).

Prints ONE JSON line.  `value` = tokens/s of chunked prefill with inputs resident in HBM;
`roofline` prices the dominant kernel (the flash forward) against the dense bf16 MFMA peak from
HIP-event timings taken inside the timed region; `decode` reports the single-token path
(16 streams, 4 cascades x 8192 slots) against HBM bandwidth; `cpu_baseline` times the CPU oracle
(the reference's eager PyTorch path restated, plus the serial update) on a bounded sample.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E
# HBM bytes per launch of the dominant kernels on the bench workloads, measured with rocprofv3 --pmc
# FETCH_SIZE and WRITE_SIZE (one pass each), each scaled by the reading for a 512 MiB device copy in the
# same run (profiles/hbm_traffic_bench_kernels.md).  Counters cannot be read inside this process.
TRAFFIC_BYTES = {"fwd_pipe_kernel": 0.220e9, "decode_stream_kernel": 2.256e9}

PREFILL = dict(B=2, H=32, KVH=8, D=128, NS=64, S=16384, C=8, Q=2048, theta=5e5, seed=2)
DECODE = dict(B=16, H=32, KVH=8, D=128, NS=64, S=32768, C=4, Q=1, theta=5e5, seed=3)


def make_cache(cfg, dtype, device):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    return CascadingKVCache(window_length=cfg["S"] // cfg["C"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"],
                            heads=cfg["KVH"], dim=cfg["D"], max_seq_len=cfg["S"], device=device, dtype=dtype,
                            cascade_func="pow2", head_reduction="mean", layers=1, eager_fill=True, verbose=False)


def chunk_pool(cfg, n, dtype, device, q_len=None, scale=1.0):
    """Seeded synthetic chunks, generated on the CPU so every run sees the same bits."""
    g = torch.Generator().manual_seed(cfg["seed"])
    B, H, KVH, D = cfg["B"], cfg["H"], cfg["KVH"], cfg["D"]
    Q = q_len or cfg["Q"]
    pool = []
    for _ in range(n):
        q = (torch.randn(B, H, Q, D, generator=g) * scale).to(dtype)
        k = (torch.randn(B, KVH, Q, D, generator=g) * scale).to(dtype)
        v = (torch.randn(B, KVH, Q, D, generator=g) * scale).to(dtype)
        pool.append((q.to(device), k.to(device), v.to(device)))
    return pool


def fill_to_steady_state(cache, cfg, pool, inv_freq):
    from cascading_kv_cache_amd.cascade_attention import cascade_attention

    need = cfg["S"] + cfg["NS"]
    done = 0
    i = 0
    while done <= need + cfg["Q"]:
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, 0, inv_freq)
        done += q.size(2)
        i += 1
    torch.cuda.synchronize()


def run_prefill(steps, warmup, dtype, device):
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    cfg = PREFILL
    cache = make_cache(cfg, dtype, device)
    inv_freq = default_inv_freq(cfg["D"], cfg["theta"], device)
    pool = chunk_pool(cfg, 4, dtype, device, scale=1.0 / math.sqrt(cfg["D"]))
    fill_to_steady_state(cache, cfg, pool, inv_freq)
    assert int(cache.mask[0].sum()) == 0, "cache must be full before the timed region"
    for i in range(warmup):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, 0, inv_freq)
    torch.cuda.synchronize()
    # timed region: only the dominant kernel is bracketed by HIP events (two records per step); an event
    # record between every pair of kernels would open a ~10 us gap each
    _abi.profile_enable(2)
    _abi.profile_read()
    t0 = time.perf_counter()
    for i in range(steps):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, 0, inv_freq)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    main_stage = _abi.profile_read()
    # untimed pass with every stage bracketed, for the per-stage table
    _abi.profile_enable(1)
    for i in range(min(steps, 10)):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, 0, inv_freq)
    torch.cuda.synchronize()
    stages = _abi.profile_read()
    _abi.profile_enable(0)

    B, H, D, Q = cfg["B"], cfg["H"], cfg["D"], cfg["Q"]
    n_cached = cfg["NS"] + cfg["S"]
    # algorithmic flops of one forward launch: QK^T and PV over the visible keys only
    flops_fwd = 4.0 * B * H * D * Q * (n_cached + (Q + 1) / 2.0)
    fwd_ms, fwd_n = main_stage["fwd"]  # from the timed region
    fwd_avg_ms = fwd_ms / max(fwd_n, 1)
    achieved = flops_fwd / (fwd_avg_ms * 1e-3) / 1e12
    stage_ms = {k: (ms / n if n else 0.0) for k, (ms, n) in stages.items()}
    attn_ms = stage_ms["prep"] + stage_ms["fwd"] + stage_ms["scores"] + stage_ms["finish"]
    res = dict(
        ms_per_step=dt / steps * 1e3,
        tokens_per_s=B * Q * steps / dt,
        roofline=dict(bound="mfma", achieved=achieved, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                      frac=achieved / PEAK_BF16_TFLOPS, traffic=TRAFFIC_BYTES["fwd_pipe_kernel"], kernel="fwd_pipe_kernel",
                      kernel_ms=fwd_avg_ms, algorithmic_tflop_per_launch=flops_fwd / 1e12),
        stage_ms=stage_ms,
        attention_tflops_all_stages=(flops_fwd + 2.0 * B * H * Q * (n_cached + Q)) / (attn_ms * 1e-3) / 1e12
        if attn_ms else None,
    )
    return res, cache, pool


def run_decode(steps, warmup, dtype, device):
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    cfg = DECODE
    cache = make_cache(cfg, dtype, device)
    inv_freq = default_inv_freq(cfg["D"], cfg["theta"], device)
    # pre-filled full: K, V ~ N(0, 1), trackers as after S + NS tokens
    g = torch.Generator(device=device).manual_seed(cfg["seed"])
    cache.key_cache[0].normal_(generator=g)
    cache.value_cache[0].normal_(generator=g)
    cache.sink_keys[0].normal_(generator=g)
    cache.sink_values[0].normal_(generator=g)
    W = cfg["S"] // cfg["C"]
    cache.stored_tokens[0].fill_(W)
    cache.stored_sinks[0].fill_(cfg["NS"])
    cache.mask[0].fill_(False)
    cache.sink_mask[0].fill_(False)
    cache.sink_pos[0].copy_(torch.arange(cfg["NS"], device=device).expand_as(cache.sink_pos[0]))
    # slot order == age order with start 0: deepest cascade holds the oldest tokens
    order = torch.arange(cfg["S"], device=device).view(cfg["C"], W).flip(0).reshape(-1)
    pos = torch.empty(cfg["S"], dtype=torch.long, device=device)
    pos[order] = torch.arange(cfg["S"], device=device)
    cache.pos[0].copy_(pos.expand_as(cache.pos[0]))
    cache.og_pos[0].copy_((pos + cfg["NS"] + 1).expand_as(cache.og_pos[0]))
    seen = cfg["S"] + cfg["NS"]
    cache.seen_tokens_by_layer[0] = seen
    cache._seen_host[0] = seen
    pool = chunk_pool(cfg, 8, dtype, device)
    for i in range(warmup):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, 0, inv_freq)
    torch.cuda.synchronize()
    # timed region: only the dominant kernel is bracketed by HIP events (two records per step); an event
    # record between every pair of kernels would open a ~10 us gap each
    _abi.profile_enable(2)
    _abi.profile_read()
    t0 = time.perf_counter()
    for i in range(steps):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, 0, inv_freq)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    main_stage = _abi.profile_read()
    # untimed pass with every stage bracketed, for the per-stage table
    _abi.profile_enable(1)
    for i in range(min(steps, 10)):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, 0, inv_freq)
    torch.cuda.synchronize()
    stages = _abi.profile_read()
    _abi.profile_enable(0)
    B, H, KVH, D = cfg["B"], cfg["H"], cfg["KVH"], cfg["D"]
    n_valid = cfg["NS"] + cfg["S"]
    es = 2
    # K and V of every visible key once, the score cache read and written once, q and out
    algo_bytes = 2.0 * B * KVH * n_valid * D * es + 2.0 * B * KVH * cfg["S"] * es + 2.0 * B * H * D * es
    stage_ms = {k: (ms / n if n else 0.0) for k, (ms, n) in stages.items()}
    timed = {k: (ms / n if n else 0.0) for k, (ms, n) in main_stage.items()}  # from the timed region
    main_ms = timed["decode"] if timed["decode"] > 0 else timed["fwd"]
    achieved = algo_bytes / (main_ms * 1e-3) / 1e9 if main_ms else 0.0
    return dict(
        workload="decode: B=16, 32q/8kv heads, head_dim 128, sink 64 + 4 cascades x 8192 slots (full), q=1",
        ms_per_step=dt / steps * 1e3,
        tokens_per_s=B * steps / dt,
        roofline=dict(bound="hbm", achieved=achieved, peak=PEAK_HBM_GBPS, unit="GB/s", frac=achieved / PEAK_HBM_GBPS,
                      traffic=TRAFFIC_BYTES["decode_stream_kernel"], kernel="decode_stream_kernel", kernel_ms=main_ms,
                      algorithmic_gb_per_launch=algo_bytes / 1e9),
        stage_ms=stage_ms,
    )


def run_cpu_baseline(cache, pool, dtype):
    """The oracle on the host: the reference's eager path restated, on a bounded sample of the
    prefill workload (same cache contents, a 64-token chunk instead of 2048)."""
    from oracle.attention import OracleCascadeAttention
    from oracle.update import OracleCache

    cfg = PREFILL
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    o = OracleCache(window_length=cfg["S"] // cfg["C"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"],
                    heads=cfg["KVH"], dim=cfg["D"], max_seq_len=cfg["S"], dtype=dtype)
    for name in ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask", "pos",
                 "og_pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks"):
        getattr(o, name).copy_(getattr(cache, name)[0].cpu())
    o.seen_tokens.fill_(int(cache._seen_host[0]))
    layer = OracleCascadeAttention(cfg["H"], cfg["KVH"], cfg["D"], rope_theta=cfg["theta"])
    q_s = 64
    q, k, v = (t[:, :, :q_s].cpu().contiguous() for t in pool[0])
    layer.query_pos = torch.arange(q_s).view(1, -1)
    layer.forward(q, k, v, o)  # untimed: first-touch of the cache copy and thread start-up
    t0 = time.perf_counter()
    reps = 0
    while True:  # a bounded sample: about ten seconds of CPU work
        layer.forward(q, k, v, o)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 256:
            break
    dt = time.perf_counter() - t0
    return dict(value=cfg["B"] * q_s * reps / dt, unit="tokens/s", cores=threads, kind="port",
                sample=f"{reps} x (2 streams x {q_s}-token chunk over the full 64+16384-slot cache), i.e. 1/32 of one "
                       f"step's tokens per repetition; eager attention + score EMA + serial update in bf16")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 512 MiB device copy, the known-size reference that scales the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU mode (every (batch, kv-head) unit is "
              "independent, so it would shard by kv head with no exchange except a per-key score reduction). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    dtype = torch.bfloat16
    pre, cache, pool = run_prefill(args.steps, args.warmup, dtype, device)
    cpu = None if args.no_cpu else run_cpu_baseline(cache, pool, dtype)
    del cache, pool
    torch.cuda.empty_cache()
    dec = None if args.no_decode else run_decode(max(args.steps, 20), args.warmup, dtype, device)
    if args.calibrate_copy:
        src = torch.ones(512 << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    line = {
        "metric": "prefill+decode tokens/s (8B-shape, C=8, 64K window); MFMA% and HBM GB/s vs peak",
        "value": pre["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": pre["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "chunked prefill, one attention layer: B=2, 32q/8kv heads, head_dim 128, sink 64 + "
                               "8 cascades x 2048 slots (full), 2048-token chunks, attention + score EMA + cache update"},
        "roofline": pre["roofline"],
        "cpu_baseline": cpu,
        "prefill_stage_ms": pre["stage_ms"],
        "prefill_attention_tflops_all_stages": pre["attention_tflops_all_stages"],
        "decode": dec,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
