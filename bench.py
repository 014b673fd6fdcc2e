#!/usr/bin/env python3
"""Throughput of the cascade attention hot path on one MI355X.

Headline workload = one attention layer of the Llama-3.1-8B shape (32 query / 8 kv heads, head_dim 128, bf16,
one stream) over a 64 sinks + 65536-slot cache split into 8 cascades (8 x 8192), the cache already full (steady
state of a long stream).  A "step" is one pass of the path in the proportions of the 131072-token prompt + 256
greedy tokens the workload is quoted on: the attention + score EMA + cache update of one 4096-token prefill
chunk, followed by 8 single-token decode steps on the same cache.  `value` = tokens (prefill + decode) per
second with every input resident in HBM.

Prints ONE JSON line.  `roofline` prices the dominant kernel (the flash forward of the prefill chunk) against
the dense bf16 MFMA peak from HIP-event timings of that kernel's own dispatch inside the timed region.  Named
sub-records carry their own roofline: `decode` (the single-token steps of the headline workload against HBM
bandwidth), `update` (the cache update of the headline chunk against HBM bandwidth, bytes counted from the
state difference), `cfg2_prefill` (B=2, 8 x 2048 slots, 2048-token chunks) and `cfg3_decode` (B=16,
4 x 8192 slots, one token) and `cfg4_full_model` (the whole 32-layer Llama-3.1-8B-shape decoder with random weights:
131072 prompt tokens in 4096-token strides, then 256 greedy tokens), `cfg5_full_model` (the Qwen2-7B-shape decoder,
B=4, 262144 tokens per stream), each checked after its stream (every layer saw every token, every ring full, position
ids a permutation, finite logits), `cfg1_gpu` (config 1, float32, on the device beside `cpu_config1`) and
`short_stride` (128- and 512-token strides on the headline cache).  `cpu_baseline` times the CPU oracle (the reference's eager PyTorch path restated,
plus the serial update) on a bounded sample of the headline workload on the box's host cores.
"""
import argparse
import hashlib
import json
import math
import os
import re
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E

LAYER = dict(name="llama3.1-8b layer, 64K window", B=1, H=32, KVH=8, D=128, NS=64, S=65536, C=8, Q=4096, theta=5e5,
             seed=4, decode_per_chunk=8, layers=4)
CFG2 = dict(name="cfg2", B=2, H=32, KVH=8, D=128, NS=64, S=16384, C=8, Q=2048, theta=5e5, seed=2)
CFG3 = dict(name="cfg3", B=16, H=32, KVH=8, D=128, NS=64, S=32768, C=4, Q=1, theta=5e5, seed=3)
# whole decoders with random weights: every layer through the library, everything else plain torch
MODEL4 = dict(name="cfg4", preset="llama3.1-8b", B=1, prompt=131072, stride=4096, window=65536, cascades=8, new=256, seed=4)
MODEL5 = dict(name="cfg5", preset="qwen2-7b", B=4, prompt=262144, stride=4096, window=32768, cascades=16, new=0, seed=5)

STATE = ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask", "pos", "og_pos",
         "sink_pos", "stored_tokens", "start_indices", "stored_sinks")


def measured_traffic(kernel, workload):
    """HBM bytes per launch of `kernel` on `workload` from the committed counter summary
    (profiles/hbm_traffic_bench_kernels.md: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy of known
    size).  Counters cannot be read inside this process, so the summary is the only source; it records the
    hash of the kernel's source file, and a figure taken from another version of that file is not reported."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_bench_kernels.md")
    try:
        text = open(path).read()
    except OSError:
        return None
    for line in text.splitlines():
        m = re.match(r"\|\s*`(\w+)`\s*\|\s*([\w.-]+)\s*\|\s*([\w./]+)\s*\|\s*([0-9a-f]{16})\s*\|\s*([0-9.]+)\s*\|\s*([0-9.]+)\s*\|", line)
        if not m or m.group(1) != kernel or m.group(2) != workload:
            continue
        src = os.path.join(ROOT, "cascading_kv_cache_amd", "csrc", m.group(3))
        try:
            digest = hashlib.sha256(open(src, "rb").read()).hexdigest()[:16]
        except OSError:
            return None
        if digest != m.group(4):
            return None  # the kernel's source changed since the counters were read
        return (float(m.group(5)) + float(m.group(6))) * 1e9
    return None


def make_cache(cfg, dtype, device):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    return CascadingKVCache(window_length=cfg["S"] // cfg["C"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"],
                            heads=cfg["KVH"], dim=cfg["D"], max_seq_len=cfg["S"], device=device, dtype=dtype,
                            cascade_func="pow2", head_reduction="mean", layers=cfg.get("layers", 1), eager_fill=True,
                            verbose=False)


def chunk_pool(cfg, n, dtype, device, q_len=None, scale=1.0, seed_offset=0):
    """Seeded synthetic chunks, generated on the CPU so every run sees the same bits."""
    g = torch.Generator().manual_seed(cfg["seed"] + seed_offset)
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
    for layer in range(cfg.get("layers", 1)):
        done = 0
        i = 0
        while done <= need + pool[0][0].size(2):
            q, k, v = pool[i % len(pool)]
            cascade_attention(q, k, v, cache, layer, inv_freq)
            done += q.size(2)
            i += 1
        torch.cuda.synchronize()
        assert int(cache.mask[layer].sum()) == 0, "cache must be full before the timed region"


def update_traffic(workload, single_token=False):
    """Measured HBM bytes of one cache update: the sum over its launches (None when any figure is stale)."""
    names = (["ckv_update_one_kernel"] if single_token else
             ["ckv_update_plan_steady_kernel", "ckv_update_plan_kernel", "ckv_update_apply_vec_kernel"])
    parts = [measured_traffic(k, workload) for k in names]
    return None if any(x is None for x in parts) else sum(parts)


def prefill_flops(cfg):
    """Algorithmic flops of one forward launch: QK^T and PV over the visible keys only (masked slots and the
    causal upper triangle excluded), 2 flop per multiply-add."""
    n_cached = cfg["NS"] + cfg["S"]
    return 4.0 * cfg["B"] * cfg["H"] * cfg["D"] * cfg["Q"] * (n_cached + (cfg["Q"] + 1) / 2.0)


def decode_bytes(cfg, es=2):
    """Algorithmic bytes of one single-token step: K and V of every visible key once, the score cache read and
    written once, q and out."""
    n_valid = cfg["NS"] + cfg["S"]
    return (2.0 * cfg["B"] * cfg["KVH"] * n_valid * cfg["D"] * es + 2.0 * cfg["B"] * cfg["KVH"] * cfg["S"] * es +
            2.0 * cfg["B"] * cfg["H"] * cfg["D"] * es)


def update_bytes(cache, cfg, k, v, new_scores, es=2):
    """Algorithmic bytes of one cache update, counted from the state difference (untimed): per (b, kv head) the
    incoming rows read once, every old row that ends in a different slot read once, every slot whose content
    differs afterwards written once (row = K, V, score, original index), plus the position ids of every slot."""
    B, KVH, D, S = cfg["B"], cfg["KVH"], cfg["D"], cfg["S"]
    q_len = k.size(2)
    before = cache.og_pos[0].clone()
    before_valid = ~cache.mask[0].clone()
    snap = {n: getattr(cache, n)[0].clone() for n in STATE}
    seen_host, seen_dev = cache._seen_host[0], cache.seen_tokens_by_layer.clone()
    cache.update_state(k, v, 0, new_scores)
    torch.cuda.synchronize()
    after = cache.og_pos[0]
    after_valid = ~cache.mask[0]
    changed = ((after != before) | (after_valid != before_valid)) & after_valid
    n_changed = int(changed.sum())
    n_reloc = 0
    for b in range(B):
        for h in range(KVH):
            moved = after[b, h][changed[b, h]]
            n_reloc += int(torch.isin(moved, before[b, h][before_valid[b, h]]).sum())
    for n, t in snap.items():  # leave the cache as it was
        getattr(cache, n)[0].copy_(t)
    cache._seen_host[0] = seen_host
    cache.seen_tokens_by_layer.copy_(seen_dev)
    row = 2 * D * es + es + 8
    total = B * KVH * q_len * (2 * D * es + es) + (n_reloc + n_changed) * row + B * KVH * S * 8
    return float(total), dict(rows_in=B * KVH * q_len, rows_relocated=n_reloc, slots_rewritten=n_changed)


def update_kernel_ms(cache, k, v, new_scores, reps=20):
    """Kernel time of one cache update: the durations of all its kernels (plan and apply launches), each timed by
    events attached to its own dispatch, summed per call.  The calls advance the (steady-state) cache."""
    from cascading_kv_cache_amd import _abi

    for _ in range(3):
        cache.update_state(k, v, 0, new_scores)
    torch.cuda.synchronize()
    _abi.profile_enable(3)
    _abi.profile_read()
    for _ in range(reps):
        cache.update_state(k, v, 0, new_scores)
    torch.cuda.synchronize()
    st = _abi.profile_read()
    _abi.profile_enable(0)
    return (st["plan"][0] + st["apply"][0]) / reps, {"plan_ms": st["plan"][0] / reps, "apply_ms": st["apply"][0] / reps,
                                                       "launches_per_call": (st["plan"][1] + st["apply"][1]) / reps}


def stage_table(stages, calls=None):
    """Milliseconds per stage: per launch of the stage, or, with `calls`, per call of the operator (a stage may
    be several launches of one call: the update plans a long chunk in pieces)."""
    return {k: (ms / (calls if calls else n) if n else 0.0) for k, (ms, n) in stages.items()}


def run_layer(steps, warmup, dtype, device):
    """The headline: per step one 4096-token chunk and 8 single-token steps on the 64K-window cache."""
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascade_attention import DecodeStepGraph, cascade_attention, default_inv_freq

    cfg = LAYER
    cache = make_cache(cfg, dtype, device)
    inv_freq = default_inv_freq(cfg["D"], cfg["theta"], device)
    pool = chunk_pool(cfg, 3, dtype, device, scale=1.0 / math.sqrt(cfg["D"]))
    dpool = chunk_pool(cfg, 8, dtype, device, q_len=1, seed_offset=100)
    fill_to_steady_state(cache, cfg, pool, inv_freq)
    n_dec = cfg["decode_per_chunk"]
    # the same steps replayed from a HIP graph are timed beside the eager launches (untimed region below): on
    # this platform a replay of the recorded kernels is not faster than launching them, so the timed region
    # launches eagerly
    graph = DecodeStepGraph(cache, 0, inv_freq, cfg["H"])
    for j in range(2):
        graph.step(*dpool[j])

    # Calls go round several layers of the same shape, as in a model: what a call left in the last-level cache
    # (256 MB; a layer's K and V are 0.27 GB) is gone when that layer is called again.  On one layer alone the
    # single-token kernel reads 6 % faster.
    n_layers = cfg["layers"]

    def step(i):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, i % n_layers, inv_freq)
        for j in range(n_dec):
            cascade_attention(*dpool[(i * n_dec + j) % len(dpool)], cache, (i + j) % n_layers, inv_freq)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    # timed region: only the two dominant kernels carry HIP events, attached to their own dispatch (an event
    # record in the stream between every pair of kernels would open a ~10 us gap each), and only every fourth
    # launch of each (a timed dispatch still costs ~6 us before and ~5 us after the kernel)
    _abi.profile_enable(4)
    _abi.profile_read()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timed = stage_table(_abi.profile_read())
    _abi.profile_enable(0)

    # untimed: the two phases apart (wall clock), then with every stage bracketed for the per-stage tables
    def phase(fn, reps):
        torch.cuda.synchronize()
        t = time.perf_counter()
        for i in range(reps):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / reps

    def one_chunk(i):
        q, k, v = pool[i % len(pool)]
        cascade_attention(q, k, v, cache, i % n_layers, inv_freq)

    def one_token(i):
        q1, k1, v1 = dpool[i % len(dpool)]
        cascade_attention(q1, k1, v1, cache, i % n_layers, inv_freq)

    def one_token_graph(i):
        graph.step(*dpool[i % len(dpool)])

    chunk_s = phase(one_chunk, max(3, min(steps, 10)))
    token_s = phase(one_token, 64)
    token_graph_s = phase(one_token_graph, 64)
    _abi.profile_enable(1)
    _abi.profile_read()
    n_pre = max(3, min(steps, 10))
    for i in range(n_pre):
        one_chunk(i)
    torch.cuda.synchronize()
    pre_stages = stage_table(_abi.profile_read(), n_pre)
    for i in range(32):
        one_token(i)
    torch.cuda.synchronize()
    dec_stages = stage_table(_abi.profile_read(), 32)
    _abi.profile_enable(0)

    B, Q = cfg["B"], cfg["Q"]
    flops = prefill_flops(cfg)
    fwd_ms = timed["fwd"]
    achieved = flops / (fwd_ms * 1e-3) / 1e12 if fwd_ms else 0.0
    attn_ms = pre_stages["prep"] + pre_stages["fwd"] + pre_stages["scores"] + pre_stages["finish"]
    n_cached = cfg["NS"] + cfg["S"]
    dec_ms = timed["decode"]
    dbytes = decode_bytes(cfg)
    dec_achieved = dbytes / (dec_ms * 1e-3) / 1e9 if dec_ms else 0.0
    # cache update of the headline chunk: bytes from the state difference, time from the stage timers
    q, k, v = pool[0]
    new_scores = torch.rand(B, cfg["KVH"], Q, device=device).mul_(1e-6).to(dtype)
    ubytes, ucount = update_bytes(cache, cfg, k, v, new_scores)
    upd_ms, upd_parts = update_kernel_ms(cache, k, v, new_scores)
    ucount.update(upd_parts)
    res = dict(
        ms_per_step=dt / steps * 1e3,
        tokens_per_s=B * (Q + n_dec) * steps / dt,
        roofline=dict(bound="mfma", achieved=achieved, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                      frac=achieved / PEAK_BF16_TFLOPS,
                      traffic=measured_traffic("fwd_pipe_kernel", "layer64k"), kernel="fwd_pipe_kernel",
                      kernel_ms=fwd_ms, algorithmic_tflop_per_launch=flops / 1e12),
        prefill=dict(tokens_per_s=B * Q / chunk_s, ms_per_chunk=chunk_s * 1e3, stage_ms=pre_stages,
                     attention_tflops_all_stages=(flops + 2.0 * B * cfg["H"] * Q * (n_cached + Q)) / (attn_ms * 1e-3) / 1e12
                     if attn_ms else None),
        decode=dict(workload="single-token steps on the headline cache (B=1, 64 sinks + 8 x 8192 slots, full)",
                    tokens_per_s=B / token_s, ms_per_step=token_s * 1e3, ms_per_step_graph_replay=token_graph_s * 1e3,
                    stage_ms=dec_stages,
                    roofline=dict(bound="hbm", achieved=dec_achieved, peak=PEAK_HBM_GBPS, unit="GB/s",
                                  frac=dec_achieved / PEAK_HBM_GBPS,
                                  traffic=measured_traffic("decode_stream_kernel", "layer64k"),
                                  kernel="decode_stream_kernel", kernel_ms=dec_ms,
                                  algorithmic_gb_per_launch=dbytes / 1e9),
                    whole_step_gbps=dbytes / token_s / 1e9),
        update=dict(workload="cache update of one 4096-token chunk into the full headline cache",
                    roofline=dict(bound="hbm", achieved=ubytes / (upd_ms * 1e-3) / 1e9 if upd_ms else 0.0,
                                  peak=PEAK_HBM_GBPS, unit="GB/s",
                                  frac=ubytes / (upd_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS if upd_ms else 0.0,
                                  traffic=update_traffic("layer64k"),
                                  kernel="ckv_update_plan_steady_kernel + ckv_update_plan_kernel + ckv_update_apply_vec_kernel",
                                  kernel_ms=upd_ms,
                                  algorithmic_gb_per_launch=ubytes / 1e9), **ucount),
    )
    return res, cache, pool


def run_cfg2(steps, warmup, dtype, device):
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    cfg = CFG2
    cache = make_cache(cfg, dtype, device)
    inv_freq = default_inv_freq(cfg["D"], cfg["theta"], device)
    pool = chunk_pool(cfg, 4, dtype, device, scale=1.0 / math.sqrt(cfg["D"]))
    fill_to_steady_state(cache, cfg, pool, inv_freq)
    for i in range(warmup):
        cascade_attention(*pool[i % len(pool)], cache, 0, inv_freq)
    torch.cuda.synchronize()
    _abi.profile_enable(4)
    _abi.profile_read()
    t0 = time.perf_counter()
    for i in range(steps):
        cascade_attention(*pool[i % len(pool)], cache, 0, inv_freq)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timed = stage_table(_abi.profile_read())
    _abi.profile_enable(1)
    for i in range(min(steps, 10)):
        cascade_attention(*pool[i % len(pool)], cache, 0, inv_freq)
    torch.cuda.synchronize()
    stages = stage_table(_abi.profile_read(), min(steps, 10))
    _abi.profile_enable(0)
    B, H, Q = cfg["B"], cfg["H"], cfg["Q"]
    flops = prefill_flops(cfg)
    fwd_ms = timed["fwd"]
    achieved = flops / (fwd_ms * 1e-3) / 1e12 if fwd_ms else 0.0
    attn_ms = stages["prep"] + stages["fwd"] + stages["scores"] + stages["finish"]
    q, k, v = pool[0]
    new_scores = torch.rand(B, cfg["KVH"], Q, device=device).mul_(1e-6).to(dtype)
    ubytes, ucount = update_bytes(cache, cfg, k, v, new_scores)
    upd_ms, upd_parts = update_kernel_ms(cache, k, v, new_scores)
    ucount.update(upd_parts)
    return dict(
        workload="chunked prefill: B=2, 32q/8kv heads, head_dim 128, sink 64 + 8 cascades x 2048 slots (full), 2048-token chunks",
        ms_per_step=dt / steps * 1e3, tokens_per_s=B * Q * steps / dt,
        roofline=dict(bound="mfma", achieved=achieved, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                      frac=achieved / PEAK_BF16_TFLOPS, traffic=measured_traffic("fwd_pipe_kernel", "cfg2"),
                      kernel="fwd_pipe_kernel", kernel_ms=fwd_ms, algorithmic_tflop_per_launch=flops / 1e12),
        stage_ms=stages,
        attention_tflops_all_stages=(flops + 2.0 * B * H * Q * (cfg["NS"] + cfg["S"] + Q)) / (attn_ms * 1e-3) / 1e12
        if attn_ms else None,
        update_roofline=dict(bound="hbm", achieved=ubytes / (upd_ms * 1e-3) / 1e9 if upd_ms else 0.0, peak=PEAK_HBM_GBPS,
                             unit="GB/s", frac=ubytes / (upd_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS if upd_ms else 0.0,
                             traffic=update_traffic("cfg2"), kernel_ms=upd_ms, algorithmic_gb_per_launch=ubytes / 1e9, **ucount),
    )


def run_cfg3(steps, warmup, dtype, device):
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascade_attention import DecodeStepGraph, cascade_attention, default_inv_freq

    cfg = CFG3
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
    graph = DecodeStepGraph(cache, 0, inv_freq, cfg["H"])
    for i in range(max(warmup, 2)):
        graph.step(*pool[i % len(pool)])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for i in range(steps):  # the same steps replayed from the recorded graph, inputs copied in per step
        graph.step(*pool[i % len(pool)])
    torch.cuda.synchronize()
    dt_graph = time.perf_counter() - t1
    # timed region: only the dominant kernel carries HIP events, attached to its own dispatch
    _abi.profile_enable(4)
    _abi.profile_read()
    t0 = time.perf_counter()
    for i in range(steps):
        cascade_attention(*pool[i % len(pool)], cache, 0, inv_freq)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timed = stage_table(_abi.profile_read())
    _abi.profile_enable(1)
    for i in range(min(steps, 10)):
        cascade_attention(*pool[i % len(pool)], cache, 0, inv_freq)
    torch.cuda.synchronize()
    stages = stage_table(_abi.profile_read(), min(steps, 10))
    _abi.profile_enable(0)
    B = cfg["B"]
    algo = decode_bytes(cfg)
    main_ms = timed["decode"] if timed["decode"] > 0 else timed["fwd"]
    achieved = algo / (main_ms * 1e-3) / 1e9 if main_ms else 0.0
    q, k, v = pool[0]
    new_scores = torch.rand(B, cfg["KVH"], 1, device=device).mul_(1e-6).to(dtype)
    ubytes, ucount = update_bytes(cache, cfg, k, v, new_scores)
    upd_ms, upd_parts = update_kernel_ms(cache, k, v, new_scores)
    ucount.update(upd_parts)
    return dict(
        workload="decode: B=16, 32q/8kv heads, head_dim 128, sink 64 + 4 cascades x 8192 slots (full), q=1",
        steps=steps, ms_per_step=dt / steps * 1e3, tokens_per_s=B * steps / dt, ms_per_step_graph_replay=dt_graph / steps * 1e3,
        roofline=dict(bound="hbm", achieved=achieved, peak=PEAK_HBM_GBPS, unit="GB/s", frac=achieved / PEAK_HBM_GBPS,
                      traffic=measured_traffic("decode_stream_kernel", "cfg3"), kernel="decode_stream_kernel",
                      kernel_ms=main_ms, algorithmic_gb_per_launch=algo / 1e9),
        stage_ms=stages,
        update_roofline=dict(bound="hbm", achieved=ubytes / (upd_ms * 1e-3) / 1e9 if upd_ms else 0.0, peak=PEAK_HBM_GBPS,
                             unit="GB/s", frac=ubytes / (upd_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS if upd_ms else 0.0,
                             traffic=update_traffic("cfg3", single_token=True), kernel_ms=upd_ms, algorithmic_gb_per_launch=ubytes / 1e9, **ucount),
    )


def run_model(cfg, device, dtype, prompt=None):
    """The full-model workloads: a random-weight decoder of the named shape streams uniform random token ids through
    in strides and then decodes greedily, every attention layer on its own layer of one cascading cache.  One short
    untimed pass (two strides, two tokens) warms the BLAS library, then the cache is reset and the whole stream
    is timed."""
    from cascading_kv_cache_amd.decoder import PRESETS, CascadeDecoder
    mcfg = PRESETS[cfg["preset"]]
    prompt = prompt or cfg["prompt"]
    model = CascadeDecoder(mcfg, dtype=dtype, device=device, seed=cfg["seed"], init_on_device=True).fuse_projections()
    g = torch.Generator().manual_seed(cfg["seed"])
    ids = torch.randint(0, mcfg.vocab_size, (cfg["B"], prompt), generator=g).to(device)
    cache = model.new_cache(cfg["window"], cfg["cascades"], batch=cfg["B"])
    stride = cfg["stride"]

    last = {}

    def stream(n_prompt, n_new):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = None
        for i in range(0, n_prompt, stride):
            logits = model(ids[:, i:i + stride], cache)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(n_new):
            logits = model(torch.argmax(logits[:, -1, :], dim=-1)[:, None], cache)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        last["logits"] = logits
        return t1 - t0, t2 - t1

    with torch.no_grad():
        stream(2 * stride, 2)
        cache.reset(verbose=False)
        tp, td = stream(prompt, cfg["new"])
    # untimed: the stream really went through every layer's cache.  Every token of the prompt and every generated
    # token was fed once; a stream longer than sinks + window leaves every slot occupied and every ring full.
    fed = prompt + cfg["new"]
    W = cfg["window"] // cfg["cascades"]
    checks = {"layers": mcfg.num_layers, "tokens_fed_per_stream": fed}
    assert cache.seen_tokens_by_layer.tolist() == [fed] * mcfg.num_layers, "a layer missed tokens"
    assert cache._seen_host == [fed] * mcfg.num_layers, "host counters out of step with the device"
    assert bool(torch.isfinite(last["logits"].float()).all()), "non-finite logits"
    if fed > cfg["window"] + 64:
        for l in range(mcfg.num_layers):
            assert not bool(cache.mask[l].any()) and not bool(cache.sink_mask[l].any()), f"layer {l}: empty slots"
            assert bool((cache.stored_tokens[l] == W).all()), f"layer {l}: a ring is not full"
            assert bool((cache.stored_sinks[l] == 64).all()), f"layer {l}: sinks"
            row = cache.pos[l][0, 0].sort().values
            assert torch.equal(row, torch.arange(cfg["window"], device=device)), f"layer {l}: position ids are not a permutation"
        checks["every_layer_full_and_consistent"] = True
    n_p, n_d = cfg["B"] * prompt, cfg["B"] * cfg["new"]
    rec = {"workload": f"{cfg['preset']} shape, {mcfg.num_layers} layers, random weights, B={cfg['B']}: {prompt} uniform random "
                       f"token ids per stream in {stride}-token strides through sink 64 + {cfg['cascades']} x "
                       f"{cfg['window'] // cfg['cascades']} slots, then {cfg['new']} greedy tokens",
           "tokens_per_s": (n_p + n_d) / (tp + td), "prefill_tokens_per_s": n_p / tp, "prefill_s": tp,
           "decode_tokens_per_s": (n_d / td) if n_d else None, "decode_ms_per_token": (td / cfg["new"] * 1e3) if n_d else None,
           "checked_after_the_stream": checks}
    if prompt != cfg["prompt"]:
        rec["truncated"] = f"prompt shortened from {cfg['prompt']} to {prompt} tokens per stream (--model-prompt)"
    del model, cache, ids, last
    torch.cuda.empty_cache()
    return rec


def host_threads():
    """Threads for the CPU leg: every core this process may use.  os.cpu_count() reports the whole host; the
    scheduler affinity and the OMP_NUM_THREADS the box exports say what this job's share is."""
    n = os.cpu_count() or 1
    try:
        n = min(n, len(os.sched_getaffinity(0)))
    except (AttributeError, OSError):
        pass
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit() and int(env) > 0:
        n = min(n, int(env))
    return n


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def run_cpu_baseline(cache, pool, dtype):
    """The oracle on the host: the reference's eager path restated, on a bounded sample of the headline
    workload (the same full cache contents, a 256-token chunk instead of 4096)."""
    from oracle.attention import OracleCascadeAttention
    from oracle.update import OracleCache

    cfg = LAYER
    threads = host_threads()
    torch.set_num_threads(threads)
    o = OracleCache(window_length=cfg["S"] // cfg["C"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"],
                    heads=cfg["KVH"], dim=cfg["D"], max_seq_len=cfg["S"], dtype=dtype)
    for name in STATE:
        getattr(o, name).copy_(getattr(cache, name)[0].cpu())
    o.seen_tokens.fill_(int(cache._seen_host[0]))
    layer = OracleCascadeAttention(cfg["H"], cfg["KVH"], cfg["D"], rope_theta=cfg["theta"])
    q_s = 256
    q, k, v = (t[:, :, :q_s].cpu().contiguous() for t in pool[0])
    layer.query_pos = torch.arange(q_s).view(1, -1)
    layer.forward(q, k, v, o)  # untimed: first-touch of the cache copy and thread start-up
    t0 = time.perf_counter()
    reps = 0
    while True:  # a bounded sample: about fifteen seconds of CPU work
        layer.forward(q, k, v, o)
        reps += 1
        if time.perf_counter() - t0 > 15.0 or reps >= 256:
            break
    dt = time.perf_counter() - t0
    return dict(value=cfg["B"] * q_s * reps / dt, unit="tokens/s", cores=threads, kind="port",
                host_cores_reported=os.cpu_count(), cpu=cpu_model(),
                sample=f"{reps} x (one {q_s}-token chunk over the full 64+65536-slot cache), i.e. 1/{cfg['Q'] // q_s} of one "
                       f"prefill chunk's tokens per repetition; eager attention + score EMA + serial update in bf16 on "
                       f"{threads} threads")


def run_cpu_config1():
    """Config 1 in full on the host (the float32 CPU case the oracle exists for): B=1, 32q/8kv heads, head_dim
    128, sink 4, window 512 in 4 cascades, 4096 tokens in chunks of 256."""
    from oracle.attention import OracleCascadeAttention
    from oracle.update import OracleCache

    torch.set_num_threads(host_threads())
    o = OracleCache(window_length=128, num_sink_tokens=4, max_batch_size=1, heads=8, dim=128, max_seq_len=512,
                    dtype=torch.float32)
    layer = OracleCascadeAttention(32, 8, 128, rope_theta=5e5)
    g = torch.Generator().manual_seed(1)
    chunks = [(torch.randn(1, 32, 256, 128, generator=g), torch.randn(1, 8, 256, 128, generator=g),
               torch.randn(1, 8, 256, 128, generator=g)) for _ in range(16)]
    t0 = time.perf_counter()
    for q, k, v in chunks:
        layer.forward(q, k, v, o)
    dt = time.perf_counter() - t0
    return dict(value=4096 / dt, unit="tokens/s", seconds=dt, cores=host_threads(), kind="port",
                sample="config 1 in full: 4096 tokens in 16 chunks of 256, float32")


def run_gpu_config1(device):
    """Config 1 on the device, beside `cpu_config1`: the same float32 stream (B=1, 32q/8kv heads, head_dim 128,
    sink 4, window 512 in 4 cascades, 4096 tokens in 16 chunks of 256) through the library's fp32-math kernels."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    cache = CascadingKVCache(window_length=128, num_sink_tokens=4, max_batch_size=1, heads=8, dim=128, max_seq_len=512,
                             device=device, dtype=torch.float32, layers=1, verbose=False)
    inv_freq = default_inv_freq(128, 5e5, device)
    g = torch.Generator().manual_seed(1)
    chunks = [tuple(torch.randn(1, h, 256, 128, generator=g).to(device) for h in (32, 8, 8)) for _ in range(16)]

    def stream():
        cache.reset(verbose=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for q, k, v in chunks:
            cascade_attention(q, k, v, cache, 0, inv_freq)
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    stream()
    dt = min(stream() for _ in range(3))
    assert cache._seen_host[0] == 4096 and not bool(cache.mask[0].any())
    return dict(value=4096 / dt, unit="tokens/s", seconds=dt, dtype="f32",
                sample="config 1 in full on the device: 4096 tokens in 16 chunks of 256, float32 (fp32-math kernels, "
                       "no matrix cores); best of 3 streams")


def run_short_strides(cache, dtype, device):
    """The headline cache (64 sinks + 8 x 8192 slots, full) fed in the short strides the reference's own latency
    script sweeps (test-latency.bash:14): per stride the time of a call, its stages, and tokens/s."""
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    cfg = LAYER
    inv_freq = default_inv_freq(cfg["D"], cfg["theta"], device)
    out = {}
    for stride in (128, 512):
        pool = chunk_pool(cfg, 4, dtype, device, q_len=stride, scale=1.0 / math.sqrt(cfg["D"]), seed_offset=200 + stride)
        n_layers = cfg["layers"]
        for i in range(4):
            cascade_attention(*pool[i % 4], cache, i % n_layers, inv_freq)
        torch.cuda.synchronize()
        reps = 32
        t0 = time.perf_counter()
        for i in range(reps):
            cascade_attention(*pool[i % 4], cache, i % n_layers, inv_freq)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / reps
        _abi.profile_enable(1)
        _abi.profile_read()
        for i in range(8):
            cascade_attention(*pool[i % 4], cache, i % n_layers, inv_freq)
        torch.cuda.synchronize()
        stages = stage_table(_abi.profile_read(), 8)
        _abi.profile_enable(0)
        out[f"stride_{stride}"] = dict(ms_per_call=dt * 1e3, tokens_per_s=cfg["B"] * stride / dt, stage_ms=stages)
    return out


def run_dense_backward(device, dtype):
    """Backward of the dense operator ``attention(q, k, v, causal, sm_scale, mask, beta)`` at the largest shape of the
    reference's own test (cascade/models/test.py:255-267: Z=2, H=32, 1024 rows, 16384 cached + 1024 chunk keys,
    head_dim 128, half of the cached keys masked): dq, dk, dv on the matrix cores.  Algorithmic work = the five matrix
    products of the backward over the visible (row, key) pairs; the kernels run seven (both recompute QK^T and
    dO V^T) over every unmasked 32-key block."""
    from cascading_kv_cache_amd import flash_attention as fa

    Z, H, n_ctx, n_kv, D = 2, 32, 1024, 16384 + 1024, 128
    g = torch.Generator(device=device).manual_seed(20)
    q, k, v, do = (torch.randn(Z, H, n, D, device=device, dtype=torch.float32, generator=g).mul_(0.5).to(dtype)
                   for n in (n_ctx, n_kv, n_kv, n_ctx))
    mask = torch.rand(n_kv - n_ctx, device=device, generator=g) > 0.5
    o, _, lse, m = fa._forward(q, k, v, True, 0.5, mask, 0.999, True)
    for _ in range(2):
        dq, dk, dv = fa._backward(q, k, v, o, lse, m, do, 0.5)
    assert all(bool(torch.isfinite(t.float()).all()) for t in (dq, dk, dv))
    reps = 10
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fa._backward(q, k, v, o, lse, m, do, 0.5)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    visible = float((~mask).sum()) + (n_ctx + 1) / 2
    flops = 5 * 2.0 * Z * H * n_ctx * visible * D
    return dict(workload=f"dq, dk, dv of the dense operator: Z={Z}, H={H}, {n_ctx} rows, {n_kv - n_ctx} cached (half "
                         f"masked) + {n_ctx} chunk keys, head_dim {D}, bf16",
                ms=dt * 1e3, algorithmic_tflop=flops / 1e12, tflops=flops / dt / 1e12, frac_of_bf16_peak=flops / dt / 2.5e15)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sub", action="store_true", help="skip the cfg2 / cfg3 sub-records")
    ap.add_argument("--no-model", action="store_true", help="skip the full-model record (cfg4)")
    ap.add_argument("--model-prompt", type=int, default=None, help="shorter prompt for the full-model records")
    ap.add_argument("--only", choices=["layer", "cfg2", "cfg3", "cfg4", "cfg5", "bwd"], default=None,
                    help="run one workload only (for profiler runs); the JSON line then carries that record alone")
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

    def calibrate():
        if args.calibrate_copy:
            src = torch.ones(512 << 20, dtype=torch.uint8, device=device)
            dst = torch.empty_like(src)
            torch.cuda.synchronize()
            dst.copy_(src)
            torch.cuda.synchronize()

    if args.only in ("cfg4", "cfg5"):
        print(json.dumps({args.only: run_model(MODEL4 if args.only == "cfg4" else MODEL5, device, dtype, args.model_prompt)}))
        return
    if args.only == "bwd":
        print(json.dumps({"dense_backward": run_dense_backward(device, dtype)}))
        return
    if args.only in ("cfg2", "cfg3"):
        rec = (run_cfg2 if args.only == "cfg2" else run_cfg3)(max(args.steps, 3), args.warmup, dtype, device)
        calibrate()
        print(json.dumps({args.only: rec}))
        return
    layer, cache, pool = run_layer(args.steps, args.warmup, dtype, device)
    sub = args.no_sub or args.only == "layer"
    short = None if sub else run_short_strides(cache, dtype, device)
    cpu = None if args.no_cpu else run_cpu_baseline(cache, pool, dtype)
    cpu1 = None if args.no_cpu else run_cpu_config1()
    del cache, pool
    torch.cuda.empty_cache()
    gpu1 = None if sub else run_gpu_config1(device)
    bwd = None if sub else run_dense_backward(device, dtype)
    torch.cuda.empty_cache()
    cfg2 = None if sub else run_cfg2(max(args.steps, 20), args.warmup, dtype, device)
    torch.cuda.empty_cache()
    cfg3 = None if sub else run_cfg3(max(args.steps, 1024), args.warmup, dtype, device)   # the configuration's 1024 steps
    torch.cuda.empty_cache()
    cfg4 = None if (sub or args.no_model) else run_model(MODEL4, device, dtype, args.model_prompt)
    cfg5 = None if (sub or args.no_model) else run_model(MODEL5, device, dtype, args.model_prompt)
    calibrate()
    cfg = LAYER
    line = {
        "metric": "prefill+decode tokens/s (8B-shape, C=8, 64K window); MFMA% and HBM GB/s vs peak",
        "value": layer["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": layer["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "one attention layer of the Llama-3.1-8B shape (B=1, 32q/8kv heads, head_dim 128, bf16) over "
                               "sink 64 + 8 cascades x 8192 slots (64K window, full): per step one 4096-token prefill chunk "
                               "and 8 single-token decode steps (the 131072 : 256 proportion of the full-model "
                               "configuration), each = attention + score EMA + cache update; successive calls go round 4 "
                               "such layers, so no call finds its layer's rows in the last-level cache",
                   "tokens_per_step": cfg["B"] * (cfg["Q"] + cfg["decode_per_chunk"])},
        # `value` is the rate of ONE attention layer (the hot path).  The same metric over the whole 32-layer
        # decoder, projections and MLP included, is cfg4_full_model below; repeated here so that nobody reads the
        # layer's figure as the model's.
        "model_level_tokens_per_s": None if cfg4 is None else {
            "llama3.1-8b_32_layers_B1_131072+256_tokens": cfg4["tokens_per_s"],
            "prefill": cfg4["prefill_tokens_per_s"], "decode": cfg4["decode_tokens_per_s"],
            "qwen2-7b_28_layers_B4_prefill": None if cfg5 is None else cfg5["prefill_tokens_per_s"]},
        "roofline": layer["roofline"],
        "cpu_baseline": cpu,
        "cpu_config1": cpu1,
        "cfg1_gpu": gpu1,
        "prefill": layer["prefill"],
        "decode": layer["decode"],
        "update": layer["update"],
        "cfg2_prefill": cfg2,
        "cfg3_decode": cfg3,
        "cfg4_full_model": cfg4,
        "cfg5_full_model": cfg5,
        "short_stride": short,
        "dense_backward": bwd,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
