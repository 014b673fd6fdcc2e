"""GPU parity of ckv_attn / ckv_attn_dense (through the C ABI) against the CPU oracle.

Tolerances (stated by the task): attention outputs within 1e-4 abs in float32 and 2e-2 abs in
bfloat16/float16; score sums are ~1e-7-scale numbers, so they are compared RELATIVE to their
magnitude with the same figures (plus one ulp of the storage dtype); cache indices, positions
and masks bit-exact.
"""
import math

import pytest
import torch

from oracle.attention import OracleCascadeAttention
from oracle.update import OracleCache

pytestmark = pytest.mark.gpu

from parity_helpers import (META, STATE, FlipLedger, assert_scores_close, check_update_against_replay, clone_oracle,
                            flip_bound, flip_margins, push_state, tol)


def make_pair(B, KVH, D, NS, W, C, dtype, func="pow2", eager=True, reduction="mean"):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    gpu = CascadingKVCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D,
                           max_seq_len=W * C, device="cuda:0", dtype=dtype, cascade_func=func,
                           head_reduction=reduction, layers=1, eager_fill=eager, verbose=False)
    cpu = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D, max_seq_len=W * C,
                      dtype=dtype, cascade_func=func, eager_fill=eager)
    return gpu, cpu


def run_teacher_forced(B, H, KVH, D, NS, W, C, Q, chunks, dtype, seed, reduction="mean", homogeneous=False,
                       eager=True, theta=5e5, std=1.0, q_last=None, do_og_pos=False, steps=None):
    """Stream chunks through the library and the oracle, the GPU cache restarting every chunk from the
    oracle's state.  Per chunk: outputs and both score inputs of the update within tolerance, metadata
    bit-exact, the library's update equal to the oracle's update run on the library's scores, K/V of every
    slot that holds the same token bit-exact, and every slot that holds a different token explained by an
    oracle margin below twice the largest score difference.  ``steps``: chunk lengths (overrides Q / chunks /
    q_last).  Returns the ledger of differing slots."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    gpu, cpu = make_pair(B, KVH, D, NS, W, C, dtype, eager=eager, reduction=reduction)
    layer = OracleCascadeAttention(H, KVH, D, rope_theta=theta, head_reduction=reduction,
                                   homogeneous_heads=homogeneous, do_og_pos=do_og_pos)
    inv_freq = default_inv_freq(D, theta, "cuda:0")
    gen = torch.Generator().manual_seed(seed)
    ledger = FlipLedger(dtype)
    if steps is None:
        steps = [q_last if (q_last is not None and c == chunks - 1) else Q for c in range(chunks)]
    for c, qn in enumerate(steps):
        q = (torch.randn(B, H, qn, D, generator=gen) * std).to(dtype)
        k = (torch.randn(B, KVH, qn, D, generator=gen) * std).to(dtype)
        v = (torch.randn(B, KVH, qn, D, generator=gen) * std).to(dtype)
        push_state(gpu, cpu)
        replay = clone_oracle(cpu)
        pre = {"og_pos": cpu.og_pos.clone(), "mask": cpu.mask.clone()}
        seen_before = int(cpu.seen_tokens)
        out_g, new_g = cascade_attention(q.cuda(), k.cuda(), v.cuda(), gpu, 0, inv_freq, head_reduction=reduction,
                                         homogeneous_heads=homogeneous, update_cache=False, do_og_pos=do_og_pos)
        scores_g = gpu.score_cache[0].cpu().clone()   # after the attention call, before the update
        gpu.update(k.cuda(), v.cuda(), 0, score_states=new_g)
        out_c = layer.forward(q, k, v, cpu)
        torch.cuda.synchronize()
        ctx = f"chunk {c} (q={qn})"
        err = (out_g.float().cpu() - out_c.float()).abs().max().item()
        assert err <= tol(dtype), f"{ctx}: out max err {err:.3e}"
        new_c = layer.last_new_scores[:, :KVH]
        eps = assert_scores_close(new_g, new_c, dtype, f"{ctx} new-token scores")
        eps = max(eps, assert_scores_close(scores_g, layer.last_score_cache, dtype, f"{ctx} score cache after attention"))
        for name in META:
            assert torch.equal(getattr(gpu, name)[0].cpu(), getattr(cpu, name)), f"{ctx}: {name}"
        # the update itself: bit-exact against the oracle's update on the same (the library's) scores
        check_update_against_replay(gpu, replay, k, v, scores_g, new_g.cpu(), ctx=ctx)
        # slots that hold the same token as in the oracle: K and V bit-exact, scores within tolerance
        og_g = gpu.og_pos[0].cpu()
        same = og_g == cpu.og_pos
        for name in ("key_cache", "value_cache"):
            g, w = getattr(gpu, name)[0].cpu(), getattr(cpu, name)
            assert torch.equal(g[same].view(torch.uint8), w[same].view(torch.uint8)), f"{ctx}: {name} of unflipped slots"
        sg, sw = gpu.score_cache[0].cpu().float(), cpu.score_cache.float()
        assert_scores_close(torch.where(same, sg, sw), sw, dtype, f"{ctx} score cache of unflipped slots")
        # slots that hold a different token: the oracle's own margin between the two must be tie-level.
        # A chunk shorter than two windows cannot evict what it has just placed in a deeper cascade, so every
        # differing slot is one tournament decided differently.
        margins = flip_margins(og_g, cpu, pre, seen_before, layer.last_score_cache, new_c)
        ledger.record(margins, eps, same.numel(), primary_only=qn < 2 * W, ctx=ctx)
    print(ledger.summary())
    return ledger


def test_config1_float32_stream():
    """The float32 benchmark case: B=1, 32q/8kv heads, D=128, sink 4, window 512 in C=4, 4096 tokens in
    chunks of 256, theta 5e5, float32."""
    led = run_teacher_forced(1, 32, 8, 128, 4, 128, 4, 256, 16, torch.float32, seed=1)
    assert led.flips == 0, f"{led.flips} of {led.compared} slots differ in og_pos (eviction decisions flipped)"


@pytest.mark.parametrize("reduction,homogeneous", [("mean", False), ("max", False), ("median", False),
                                                   ("mean", True), ("max", True), ("median", True)])
def test_small_float32_reductions(reduction, homogeneous):
    led = run_teacher_forced(2, 6, 2, 16, 3, 8, 4, 12, 10, torch.float32, seed=2, reduction=reduction,
                             homogeneous=homogeneous, eager=False, theta=1e4)
    assert led.flips == 0


def test_ragged_last_chunk_and_decode_steps_float32():
    assert run_teacher_forced(1, 4, 2, 32, 4, 16, 2, 10, 6, torch.float32, seed=3, q_last=3).flips == 0
    assert run_teacher_forced(2, 4, 4, 64, 2, 8, 2, 1, 40, torch.float32, seed=4).flips == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_config1_shaped_sixteen_bit_stream(dtype):
    """The float32 benchmark case in the 16-bit formats: B=1, 32q/8kv heads, D=128, sink 4, window 512 in C=4,
    4096 tokens in chunks of 256, theta 5e5; the number of slots that hold another token than the oracle's is
    printed and bounded."""
    led = run_teacher_forced(1, 32, 8, 128, 4, 128, 4, 256, 16, dtype, seed=1)
    assert led.flips <= flip_bound(led), led.summary()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sixteen_bit_stream(dtype):
    led = run_teacher_forced(2, 8, 2, 128, 8, 64, 4, 64, 8, dtype, seed=5, std=0.5)
    # 16-bit scores tie or differ in the last place all the time, so a few decisions go the other way; each one
    # is checked against the oracle's margin inside run_teacher_forced, and their number is bounded (flip_bound)
    assert led.flips <= flip_bound(led), led.summary()


REDUCTIONS = [("max", False), ("median", False), ("mean", True), ("max", True), ("median", True)]


@pytest.mark.parametrize("H,KVH,Q,W,C,NS,eager,dtype,reduction,homogeneous", [
    (8, 2, 128, 256, 4, 64, True, torch.bfloat16, "mean", False),     # G = 4, the Llama grouping
    (14, 2, 96, 128, 4, 64, True, torch.bfloat16, "mean", False),     # G = 7, the Qwen2 grouping
    (4, 4, 200, 128, 2, 8, False, torch.bfloat16, "mean", False),     # G = 1, ragged chunk, sparse fill
    (16, 2, 64, 64, 8, 64, True, torch.float16, "mean", False),       # G = 8
    (8, 2, 300, 128, 4, 64, False, torch.bfloat16, "mean", False),    # chunk longer than two cascade windows
] + [(8, 2, 128, 256, 4, 64, True, torch.bfloat16, r, h) for r, h in REDUCTIONS]     # cascade_attention.py:231-248
  + [(14, 2, 96, 128, 4, 64, False, torch.float16, r, h) for r, h in REDUCTIONS])
def test_mfma_prefill_head128(H, KVH, Q, W, C, NS, eager, dtype, reduction, homogeneous):
    """head_dim 128 in 16-bit takes the MFMA kernels: stream chunks while the cache fills up and
    starts evicting, teacher-forced against the oracle, for every head reduction and both head modes."""
    led = run_teacher_forced(2, H, KVH, 128, NS, W, C, Q, 8, dtype, seed=11, eager=eager, std=0.7,
                             q_last=Q - 37, reduction=reduction, homogeneous=homogeneous)
    assert led.flips <= flip_bound(led), led.summary()


@pytest.mark.parametrize("seed", range(10))
def test_random_head128_streams(seed):
    """Random shapes on the matrix-core and single-token kernels: heads per kv head 1, 2, 4, 7 or 8, ragged
    chunk lengths from one token to several hundred mixed in one stream, windows from a few tiles to a few
    thousand slots, with and without eager fill, every head reduction."""
    import random

    rng = random.Random(1000 + seed)
    G = rng.choice([1, 2, 4, 7, 8])
    KVH = rng.choice([1, 2, 4])
    B = rng.choice([1, 2])
    W = rng.choice([16, 64, 200, 512, 1024])
    C = rng.choice([1, 2, 4, 8])
    NS = rng.choice([3, 4, 64])   # the reference's prologue needs at least one sink (cascade_attention.py:145-148)
    dtype = rng.choice([torch.bfloat16, torch.float16])
    eager = rng.random() < 0.6
    reduction = rng.choice(["mean", "max", "median"])
    homogeneous = rng.random() < 0.25
    total = NS + W * C
    steps, done = [], 0
    while done < total + 2 * W and len(steps) < 24:
        kind = rng.random()
        q = 1 if kind < 0.35 else (rng.randint(2, 40) if kind < 0.5 else rng.randint(41, max(64, min(700, total // 2))))
        steps.append(q)
        done += q
    big = steps.index(max(steps))   # the reference sizes its query positions by the first chunk (cascade_attention.py:120-123)
    steps[0], steps[big] = steps[big], steps[0]
    print(f"seed={seed} B={B} H={G * KVH} KVH={KVH} W={W} C={C} NS={NS} {dtype} eager={eager} {reduction} "
          f"homogeneous={homogeneous} steps={steps}", flush=True)
    led = run_teacher_forced(B, G * KVH, KVH, 128, NS, W, C, 0, 0, dtype, seed=seed, reduction=reduction,
                             homogeneous=homogeneous, eager=eager, std=0.7, steps=steps)
    assert led.flips <= flip_bound(led), led.summary()


@pytest.mark.parametrize("H,KVH,Q,W,C,dtype,eager", [
    (8, 2, 320, 1024, 4, torch.bfloat16, True),     # 10 workgroups' worth of rows against 4160 slots: 4 shares
    (14, 2, 256, 512, 8, torch.float16, False),     # G = 7
    (4, 4, 512, 2048, 2, torch.bfloat16, True),     # G = 1
])
def test_mfma_prefill_short_chunks_split_the_keys(H, KVH, Q, W, C, dtype, eager):
    """Short chunks of one or two streams against a few thousand slots: too few query rows to fill the chip, so the
    forward kernel deals the key tiles of a query tile out over several workgroups and a second kernel merges their
    shares.  The stream runs from the empty cache (shares without a visible key) until the cascades evict."""
    chunks = (64 + W * C) // Q + 3
    led = run_teacher_forced(1, H, KVH, 128, 64, W, C, Q, chunks, dtype, seed=31, eager=eager, std=0.7, q_last=Q - 11)
    assert led.flips <= flip_bound(led), led.summary()


@pytest.mark.parametrize("dtype,std", [(torch.bfloat16, 0.05), (torch.bfloat16, 1.0), (torch.bfloat16, 3.0),
                                       (torch.float16, 2.5), (torch.bfloat16, 6.0)])
def test_mfma_prefill_wide_range_of_logits(dtype, std):
    """With every value row equal to one the output is one whatever the logits are: the sums of a row
    and its weighted values must stay relative to the same reference while that reference moves.  Logits
    of tens of units make the running maximum of a row outgrow its reference again and again along the
    keys (the oracle is no yardstick there: its 16-bit rotation moves such logits by whole units)."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    B, H, KVH, D, NS, W, C, Q = 1, 8, 2, 128, 8, 128, 4, 96
    cache = CascadingKVCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D,
                             max_seq_len=W * C, device="cuda:0", dtype=dtype, layers=1, verbose=False)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(31)
    for c in range(9):
        q = (torch.randn(B, H, Q, D, generator=gen) * std).to(dtype).cuda()
        k = (torch.randn(B, KVH, Q, D, generator=gen) * std).to(dtype).cuda()
        # keys that grow along the chunk: later tiles hold the larger logits
        k = k * torch.linspace(0.25, 1.0, Q, device="cuda:0").to(dtype).view(1, 1, Q, 1)
        v = torch.ones(B, KVH, Q, D, dtype=dtype, device="cuda:0")
        out, new_scores = cascade_attention(q, k, v, cache, 0, inv_freq)
        torch.cuda.synchronize()
        err = (out.float() - 1.0).abs().max().item()
        assert err <= 1e-2, f"chunk {c}: rows of probabilities sum to 1 +- {err:.3e}"
        assert torch.isfinite(new_scores.float()).all() and torch.isfinite(cache.score_cache[0].float()).all()


@pytest.mark.parametrize("H,KVH,W,C,NS,eager,dtype,reduction,homogeneous", [
    (8, 2, 64, 4, 8, True, torch.bfloat16, "mean", False),      # G = 4: the streaming kernel
    (14, 2, 32, 4, 4, False, torch.bfloat16, "mean", False),    # G = 7: the streaming kernel for 5 to 8 heads
    (4, 4, 32, 2, 4, True, torch.float16, "mean", False),       # G = 1
    (16, 2, 16, 8, 64, True, torch.bfloat16, "mean", False),    # G = 8
    (8, 4, 64, 2, 6, True, torch.float32, "mean", False),       # G = 2, float32
    (8, 4, 64, 2, 6, True, torch.float32, "median", True),
] + [(8, 2, 64, 4, 8, True, torch.bfloat16, r, h) for r, h in REDUCTIONS]       # cascade_attention.py:231-248
  + [(14, 2, 32, 4, 4, False, torch.float16, r, h) for r, h in REDUCTIONS])
def test_decode_head128(H, KVH, W, C, NS, eager, dtype, reduction, homogeneous):
    """q == 1 with head_dim 128 takes the bandwidth-bound decode kernels: fill part of the cache
    with a few chunks, then run single-token steps (cache still filling, then evicting), for every head
    reduction and both head modes."""
    steps = [W * C // 2 + NS, 17] + [1] * (W * C // 2 + 40)
    led = run_teacher_forced(2, H, KVH, 128, NS, W, C, None, None, dtype, seed=21, eager=eager, std=0.7, steps=steps,
                             reduction=reduction, homogeneous=homogeneous)
    if dtype == torch.float32:
        assert led.flips == 0, led.summary()
    else:
        assert led.flips <= flip_bound(led), led.summary()


@pytest.mark.parametrize("H,KVH,dtype,fill", [
    (32, 8, torch.bfloat16, 3000),   # G = 4, cache partly filled: hidden slots inside most tiles
    (32, 8, torch.bfloat16, 6000),   # G = 4, cache full and evicting
    (16, 8, torch.float16, 2500),    # G = 2
    (8, 8, torch.bfloat16, 3500),    # G = 1
    (56, 8, torch.bfloat16, 3000),   # G = 7 (the kernel for 5 to 8 heads per kv head), partly filled
    (56, 8, torch.float16, 6000),    # G = 7, full and evicting
    (64, 8, torch.bfloat16, 2500),   # G = 8
])
def test_decode_streaming_many_items(H, KVH, dtype, fill):
    """Decode over a few thousand slots with 16 (batch, kv-head) units: more (tile, unit) items than
    workgroups, so a workgroup walks several items and crosses key-tile boundaries.  The cache is
    filled through the oracle's update alone (random keys, values and scores), and the hidden slots of
    the GPU copy are poisoned with NaN: nothing of a hidden slot may reach the output."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    B, D, NS, W, C = 2, 128, 4, 1024, 4
    gpu, cpu = make_pair(B, KVH, D, NS, W, C, dtype)
    layer = OracleCascadeAttention(H, KVH, D, rope_theta=5e5)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(5)
    done = 0
    while done < fill:
        n = min(512, fill - done)
        k = (torch.randn(B, KVH, n, D, generator=gen) * 0.7).to(dtype)
        v = (torch.randn(B, KVH, n, D, generator=gen) * 0.7).to(dtype)
        s = torch.rand(B, KVH, n, generator=gen).to(dtype)
        cpu.update(k, v, s)
        done += n
    layer.query_pos = torch.arange(0, 512, dtype=torch.long).view(1, -1)  # what a first prefill chunk leaves behind
    for step in range(3):
        q = (torch.randn(B, H, 1, D, generator=gen) * 0.7).to(dtype)
        k = (torch.randn(B, KVH, 1, D, generator=gen) * 0.7).to(dtype)
        v = (torch.randn(B, KVH, 1, D, generator=gen) * 0.7).to(dtype)
        push_state(gpu, cpu)
        hidden = gpu.mask[0].bool().expand(gpu.key_cache[0].shape[:-1])
        gpu.key_cache[0][hidden] = float("nan")
        gpu.value_cache[0][hidden] = float("nan")
        out_g, new_g = cascade_attention(q.cuda(), k.cuda(), v.cuda(), gpu, 0, inv_freq)
        out_c = layer.forward(q, k, v, cpu)
        torch.cuda.synchronize()
        assert torch.isfinite(out_g.float()).all(), f"step {step}: a hidden slot leaked into the output"
        err = (out_g.float().cpu() - out_c.float()).abs().max().item()
        assert err <= tol(dtype), f"step {step}: out max err {err:.3e}"
        assert_scores_close(new_g, layer.last_new_scores[:, :KVH], dtype, f"step {step} new-token scores")
        for name in META:
            assert torch.equal(getattr(gpu, name)[0].cpu(), getattr(cpu, name)), f"step {step}: {name}"


@pytest.mark.parametrize("dtype,D,H,KVH,Q,q_last", [
    (torch.float32, 32, 4, 2, 10, 3),       # fp32-math kernels
    (torch.bfloat16, 128, 8, 2, 64, 17),    # matrix-core prefill, key positions per (batch, kv head)
    (torch.float16, 128, 4, 4, 40, None),
    (torch.bfloat16, 128, 8, 2, 1, None),   # single-token steps, positions per (batch, kv head)
    (torch.float16, 128, 7, 1, 1, None),
])
def test_original_position_mode(dtype, D, H, KVH, Q, q_last):
    """cascade_attention.py:141-144, 161-164 (do_og_pos): cached keys are rotated per (batch, head) at the index
    of the token a slot holds; without eager fill the heads soon keep different tokens."""
    chunks = 40 if Q == 1 else 8
    led = run_teacher_forced(2, H, KVH, D, 4, 16, 2, Q, chunks, dtype, seed=21, eager=False, std=0.7,
                             q_last=q_last, do_og_pos=True)
    if dtype == torch.float32:
        assert led.flips == 0, led.summary()


@pytest.mark.parametrize("eager", [False, True])
@pytest.mark.parametrize("do_og_pos", [False, True])
def test_chunk_positions_kernel(do_og_pos, eager):
    """Position ids of a chunk against the rule of cascade_attention.py:114-150: 0.. on the first call,
    then one past the largest position id among sinks and slots (stale entries included).  ckv_chunk_positions
    computes them on the device; with eager fill (and compact ids) the host derives them from its token counter."""
    from cascading_kv_cache_amd.cascade_attention import chunk_positions

    B, KVH, D, NS, W, C = 2, 2, 32, 4, 16, 4
    gpu, cpu = make_pair(B, KVH, D, NS, W, C, torch.float32, eager=eager)
    gen = torch.Generator().manual_seed(3)
    assert torch.equal(chunk_positions(gpu, 0, 7, do_og_pos).cpu(), torch.arange(7))
    for n in (3, 9, 40, 1, 100):
        k = torch.randn(B, KVH, n, D, generator=gen)
        cpu.update(k, k.clone(), torch.rand(B, KVH, n, generator=gen))
        push_state(gpu, cpu)
        if do_og_pos:
            key_max = cpu.og_pos.amax()
        else:
            shift = NS if int(cpu.seen_tokens) > NS else 0
            key_max = cpu.pos[0, 0].amax() + shift
        want = torch.arange(5) + max(int(key_max), int(cpu.sink_pos[0, 0].amax())) + 1
        assert torch.equal(chunk_positions(gpu, 0, 5, do_og_pos).cpu(), want)


def dense_reference(q, k, v, mask, sm_scale):
    n_ctx, n_kv = q.size(2), k.size(2)
    logits = torch.matmul(q.float(), k.float().transpose(2, 3)) * sm_scale
    full = torch.cat((mask[None, :].expand(n_ctx, -1),
                      torch.ones(n_ctx, n_ctx, dtype=torch.bool, device=q.device).triu(1)), dim=-1)
    logits = logits.masked_fill(full, float("-inf"))
    p = torch.softmax(logits, dim=-1)
    return torch.matmul(p, v.float()), p


@pytest.mark.parametrize("Z,H,N_CTX,N_KV,HEAD_DIM", [
    (1, 2, 128, 128, 64), (1, 2, 256, 256, 64), (1, 1, 128, 128 + 128, 64), (1, 2, 512, 2560, 64),
    (1, 2, 500, 2048 + 500, 64), (1, 2, 500, 2048 + 64 + 500, 64), (2, 4, 256, 1024 + 256, 128),
    # head_dim 128 in 16-bit runs on the matrix-core kernels: ragged sizes, no cache at all, long cache
    (1, 2, 500, 2048 + 64 + 500, 128), (2, 3, 384, 384, 128), (1, 2, 130, 4096 + 130, 128),
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_dense_operator_forward(Z, H, N_CTX, N_KV, HEAD_DIM, dtype):
    """The forward half of cascade/models/test.py:177-269: seed 20, N(0, 0.5) inputs, sm_scale 0.5,
    random cache mask, atol 1e-2 (1e-4 in float32)."""
    from cascading_kv_cache_amd.flash_attention import attention

    torch.manual_seed(20)
    q = torch.empty((Z, H, N_CTX, HEAD_DIM), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5)
    k = torch.empty((Z, H, N_KV, HEAD_DIM), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5)
    v = torch.empty((Z, H, N_KV, HEAD_DIM), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5)
    mask = torch.rand(N_KV - N_CTX, device="cuda") > 0.5
    ref, p = dense_reference(q, k, v, mask, 0.5)
    out, scores = attention(q, k, v, True, 0.5, mask, 0.9999)
    atol = 1e-4 if dtype == torch.float32 else 1e-2
    assert (out.float() - ref).abs().max().item() <= atol
    # exact version of what cascade/models/test.py:271-318 only rank-correlates
    w = (1 - 0.9999) * 0.9999 ** torch.arange(N_CTX - 1, -1, -1, device="cuda", dtype=torch.float64)
    want = (p.double() * w[None, None, :, None]).sum(dim=2)
    assert_scores_close(scores, want, dtype, "dense scores")


def test_attention_rejects_cpu_tensors():
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.flash_attention import attention

    q = torch.zeros(1, 1, 16, 64)
    with pytest.raises(_abi.CkvError):
        attention(q, q, q, True, 1.0, torch.zeros(0, dtype=torch.bool), 0.9)


@pytest.mark.parametrize("Z,H,N_CTX,N_KV,HEAD_DIM", [
    (1, 2, 128, 128, 64), (1, 2, 256, 256, 64), (1, 2, 512, 512, 64), (1, 1, 128, 128 + 128, 64),
    (1, 2, 1024, 16384 + 1024, 64), (2, 32, 1024, 16384 + 1024, 128), (1, 2, 512, 2560, 64),
    (1, 2, 500, 2048 + 500, 64), (1, 2, 500, 2048 + 64 + 500, 64), (2, 3, 77, 300 + 77, 32),
    (1, 3, 90, 200 + 90, 16),   # the smallest head size the operator takes
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_dense_operator_backward(Z, H, N_CTX, N_KV, HEAD_DIM, dtype):
    """The backward half of cascade/models/test.py:177-269: seed 20, N(0, 0.5) inputs, sm_scale 0.5, random cache
    mask; dq, dk, dv of the operator against autograd through the dense formula (softmax in float32, then the
    product with v in the tensor dtype), atol 1e-2 in float16 as in the reference's test, 1e-4 in float32, 2e-2 in
    bfloat16 plus two units in the last place of the value (gradients of a key seen by hundreds of rows reach
    magnitudes of 4 to 8, where neighbouring bfloat16 values are 3e-2 apart, and the reference formula rounds P
    and the products to bfloat16 where the kernels round once)."""
    torch.manual_seed(20)
    q = torch.empty((Z, H, N_CTX, HEAD_DIM), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5).requires_grad_()
    k = torch.empty((Z, H, N_KV, HEAD_DIM), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5).requires_grad_()
    v = torch.empty((Z, H, N_KV, HEAD_DIM), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5).requires_grad_()
    mask = torch.rand(N_KV - N_CTX, device="cuda") > 0.5
    check_backward_against_autograd(q, k, v, mask, dtype)


def check_backward_against_autograd(q, k, v, mask, dtype, sm_scale=0.5):
    """dq, dk, dv of ``attention`` against autograd through the dense formula; q, k, v are leaves."""
    from cascading_kv_cache_amd.flash_attention import attention

    N_CTX, N_KV = q.size(2), k.size(2)
    full = torch.cat((mask[None, :].expand(N_CTX, -1),
                      torch.ones(N_CTX, N_CTX, dtype=torch.bool, device="cuda").triu(1)), dim=-1)
    dout = torch.randn_like(q)
    p = torch.matmul(q, k.transpose(2, 3)) * sm_scale
    p = p.masked_fill(full, float("-inf"))
    p = torch.softmax(p.float(), dim=-1).to(dtype)
    ref_out = torch.matmul(p, v).to(dtype)
    ref_out.backward(dout)
    ref_dv, v.grad = v.grad.clone(), None
    ref_dk, k.grad = k.grad.clone(), None
    ref_dq, q.grad = q.grad.clone(), None
    del p
    out, scores = attention(q, k, v, True, sm_scale, mask, 1.0)
    assert not scores.requires_grad
    atol = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 2e-2}[dtype]
    assert (out.float() - ref_out.float()).abs().max().item() <= atol
    out.backward(dout, None)
    for name, got, want in (("dv", v.grad, ref_dv), ("dk", k.grad, ref_dk), ("dq", q.grad, ref_dq)):
        assert got.shape == want.shape and got.dtype == want.dtype
        rtol = 2.0 ** -6 if dtype == torch.bfloat16 else 0.0
        excess = ((got.float() - want.float()).abs() - rtol * want.float().abs()).max().item()
        assert excess <= atol, f"{name}: error exceeds the relative allowance by {excess:.3e}"
    # a masked slot receives no gradient at all
    if int(mask.sum()) > 0:
        assert k.grad[:, :, : N_KV - N_CTX][:, :, mask].abs().max().item() == 0.0
        assert v.grad[:, :, : N_KV - N_CTX][:, :, mask].abs().max().item() == 0.0


@pytest.mark.parametrize("Z,H,N_CTX,N_KV", [
    (1, 2, 128, 128), (1, 2, 100, 100), (1, 1, 128, 128 + 128), (1, 2, 500, 2048 + 64 + 500), (2, 3, 77, 300 + 77),
    (1, 2, 33, 1 + 33), (1, 1, 1, 40 + 1), (1, 2, 260, 95 + 260),
])
@pytest.mark.parametrize("masking", ["random", "none", "stretches"])
@pytest.mark.parametrize("layout", ["heads_first", "tokens_first"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_backward_on_the_matrix_cores(Z, H, N_CTX, N_KV, masking, layout, dtype):
    """head_dim 128 in the 16-bit formats runs the backward on the matrix cores (32-row blocks, 128 stationary rows
    per workgroup): sizes that are no multiple of either, cached stretches that end inside a block, no cached keys
    at all, whole blocks of masked keys, and tensors laid out (batch, tokens, heads, dim) as projections leave them."""
    torch.manual_seed(21)
    D = 128

    def leaf(n):
        if layout == "heads_first":
            t = torch.empty((Z, H, n, D), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5)
        else:
            t = torch.empty((Z, n, H, D), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5).transpose(1, 2)
        return t.requires_grad_()

    q, k, v = leaf(N_CTX), leaf(N_KV), leaf(N_KV)
    n_cached = N_KV - N_CTX
    if masking == "random":
        mask = torch.rand(n_cached, device="cuda") > 0.5
    elif masking == "none":
        mask = torch.zeros(n_cached, dtype=torch.bool, device="cuda")
    else:  # whole 32-key blocks hidden, and a stretch that starts and ends inside blocks
        mask = torch.zeros(n_cached, dtype=torch.bool, device="cuda")
        mask[: min(96, n_cached)] = True
        mask[min(130, n_cached): min(171, n_cached)] = True
    check_backward_against_autograd(q, k, v, mask, dtype)


@pytest.mark.parametrize("flavour", ["llama", "qwen2"])
def test_reference_mixin_surface(flavour):
    """A layer written the way the reference's model files use the mixin — ``get_vals``, ``self.rope`` on queries,
    chunk keys, sinks and cached keys, ``repeat_kv``, then ``self.cascade_attn_flash`` / ``cascade_attn_eager``
    (cascade_attention.py:103-200) — against the fused operator on a second cache: outputs within tolerance,
    score cache within tolerance, cache metadata bit-exact, over chunks that fill the cache and evict."""
    from types import SimpleNamespace

    from cascading_kv_cache_amd.cascade_attention import (LlamaCascadeAttention, Qwen2CascadeAttention,
                                                          cascade_attention, default_inv_freq)
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    B, H, KVH, D, NS, W, C, dtype = 2, 8, 2, 128, 4, 32, 2, torch.bfloat16
    base = Qwen2CascadeAttention if flavour == "qwen2" else LlamaCascadeAttention

    class Layer(base):
        def __init__(self):
            super().__init__()
            self.num_heads, self.num_key_value_heads, self.head_dim, self.layer_idx = H, KVH, D, 0
            self.num_key_value_groups = H // KVH
            self.rope_theta, self.max_position_embeddings = 5e5, 512
            self.config = SimpleNamespace(_head_reduction="mean", _homogeneous_heads=False, _do_og_pos=False)

    def expand(x):  # repeat_kv
        return x[:, :, None].expand(-1, -1, H // KVH, -1, -1).reshape(x.size(0), H, x.size(2), x.size(3))

    layer = Layer()
    caches = [CascadingKVCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D,
                               max_seq_len=W * C, device="cuda:0", dtype=dtype, layers=1, verbose=False)
              for _ in range(2)]
    by_hand, fused = caches
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(77)
    for c, qn in enumerate((24, 24, 24, 24, 1, 1)):
        q = (torch.randn(B, H, qn, D, generator=gen) * 0.7).to(dtype).cuda()
        k = (torch.randn(B, KVH, qn, D, generator=gen) * 0.7).to(dtype).cuda()
        v = (torch.randn(B, KVH, qn, D, generator=gen) * 0.7).to(dtype).cuda()
        # teacher forcing: the hand-driven cache restarts from the fused one's state
        for name in STATE:
            getattr(by_hand, name)[0].copy_(getattr(fused, name)[0])
        by_hand.seen_tokens_by_layer.copy_(fused.seen_tokens_by_layer)
        by_hand.sync_host_counter()
        first = by_hand._seen_host[0] == 0
        sink_k, sink_v, sink_pos, sink_mask, ck, cv, key_pos, key_mask, _ = by_hand.get_vals(0)
        top = 0 if first else int(max(sink_pos.max(), key_pos.max())) + 1
        q_pos = torch.arange(top, top + qn, device="cuda:0").view(1, -1)
        q_rot, _, _ = layer.rope(q, q_pos)
        k_rot, _, _ = layer.rope(k, q_pos)
        sink_rot, _, _ = layer.rope(sink_k, sink_pos)
        cache_rot, _, _ = layer.rope(ck, key_pos)
        arm = layer.cascade_attn_flash if c % 2 == 0 else layer.cascade_attn_eager
        out_h, _ = arm(q_rot, k, v, expand(k_rot), expand(cv), expand(sink_rot), expand(sink_v), expand(cache_rot),
                       sink_mask, key_mask, first, by_hand, 1 / math.sqrt(D), qn, False)
        assert layer.last_attn_called == ("flash" if c % 2 == 0 else "eager") and layer.last_q_size == qn
        out_f, _ = cascade_attention(q, k, v, fused, 0, inv_freq)
        torch.cuda.synchronize()
        err = (out_h.float() - out_f.float()).abs().max().item()
        assert err <= tol(dtype), f"chunk {c}: out differs by {err:.3e}"
        for name in META:
            assert torch.equal(getattr(by_hand, name)[0], getattr(fused, name)[0]), f"chunk {c}: {name}"
        assert by_hand._seen_host == fused._seen_host
        same = by_hand.og_pos[0] == fused.og_pos[0]
        assert same.float().mean().item() >= 0.99, f"chunk {c}: {(~same).sum().item()} slots hold another token"
        sh, sf = by_hand.score_cache[0].float(), fused.score_cache[0].float()
        assert_scores_close(torch.where(same, sh, sf), sf, dtype, f"chunk {c}: score cache")


def test_backward_is_refused_up_front_for_head_sizes_it_does_not_tile():
    """head_dim 256 runs forward (the reference operator's set is 16 .. 256) but the backward kernels stage fp32
    rows of at most 192 columns: asking for gradients raises at the call, not later inside ``.backward()``; head
    sizes that are not a multiple of 16 never reach the operator (flash_attention.py:545-551), and the C entry point
    refuses them too."""
    import ctypes as C

    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.flash_attention import attention

    q = torch.randn(1, 1, 32, 256, device="cuda", dtype=torch.float16)
    k = torch.randn(1, 1, 48, 256, device="cuda", dtype=torch.float16)
    mask = torch.zeros(16, dtype=torch.bool, device="cuda")
    out, _ = attention(q, k, k.clone(), True, 0.1, mask, 1.0)          # inference: fine
    assert out.shape == q.shape and bool(torch.isfinite(out.float()).all())
    with pytest.raises(_abi.CkvError):
        attention(q.clone().requires_grad_(), k, k.clone(), True, 0.1, mask, 1.0)
    g = _abi.DenseBwdArgs()
    g.dtype = _abi.CKV_F16
    g.B, g.H, g.n_ctx, g.n_kv, g.D = 1, 1, 16, 32, 72
    assert _abi.lib().ckv_attn_dense_bwd(C.byref(g), None) == -6       # CKV_ERR_UNSUPPORTED


@pytest.mark.parametrize("D,dtype", [(80, torch.float16), (192, torch.bfloat16), (192, torch.float32), (48, torch.float32)])
def test_backward_head_sizes_outside_the_reference_set(D, dtype):
    """The C entry points take head sizes the reference operator does not (any multiple of 16 up to 192 backward):
    forward and backward of the dense operator, called below the operator's own shape check, against autograd
    through the dense formula."""
    from cascading_kv_cache_amd import flash_attention as fa

    torch.manual_seed(21)
    Z, H, N_CTX, N_KV = 1, 2, 70, 150 + 70
    q = torch.empty((Z, H, N_CTX, D), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5).requires_grad_()
    k = torch.empty((Z, H, N_KV, D), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5).requires_grad_()
    v = torch.empty((Z, H, N_KV, D), dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5).requires_grad_()
    mask = torch.rand(N_KV - N_CTX, device="cuda") > 0.5
    full = torch.cat((mask[None, :].expand(N_CTX, -1),
                      torch.ones(N_CTX, N_CTX, dtype=torch.bool, device="cuda").triu(1)), dim=-1)
    sm_scale = 1.0 / math.sqrt(D)
    dout = torch.randn_like(q)
    p = (torch.matmul(q, k.transpose(2, 3)) * sm_scale).masked_fill(full, float("-inf"))
    ref_out = torch.matmul(torch.softmax(p.float(), dim=-1).to(dtype), v)
    ref_out.backward(dout)
    with torch.no_grad():
        out, _, lse, m = fa._forward(q, k, v, True, sm_scale, mask, 1.0, True)
        dq, dk, dv = fa._backward(q, k, v, out, lse, m, dout, sm_scale)
    atol = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 2e-2}[dtype]
    assert (out.float() - ref_out.float()).abs().max().item() <= atol
    for name, got, want in (("dv", dv, v.grad), ("dk", dk, k.grad), ("dq", dq, q.grad)):
        rtol = 2.0 ** -6 if dtype == torch.bfloat16 else 0.0
        excess = ((got.float() - want.float()).abs() - rtol * want.float().abs()).max().item()
        assert excess <= atol, f"{name}: error exceeds the allowance by {excess:.3e}"


@pytest.mark.parametrize("dtype,H,KVH", [(torch.bfloat16, 8, 2), (torch.float16, 14, 2), (torch.float32, 8, 2)])
def test_filled_slots_hint_changes_nothing(dtype, H, KVH):
    """``ckv_attn_args.filled_slots`` is a hint, never a second mask: single-token steps on a cache that is still
    filling give bit-identical outputs, scores and score cache whether the caller passes the hint (the host wrapper
    does, from its token counter) or not (``replayable=True`` leaves it out) -- on the streaming kernels, which use
    it to skip empty tiles, and on the paths that ignore it."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    B, D, NS, W, C = 2, 128, 4, 256, 4
    with_hint, without = (make_pair(B, KVH, D, NS, W, C, dtype)[0] for _ in range(2))
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(31)
    q = (torch.randn(B, H, 150, D, generator=gen) * 0.7).to(dtype).cuda()
    k = (torch.randn(B, KVH, 150, D, generator=gen) * 0.7).to(dtype).cuda()
    v = (torch.randn(B, KVH, 150, D, generator=gen) * 0.7).to(dtype).cuda()
    for c in (with_hint, without):
        cascade_attention(q, k, v, c, 0, inv_freq)         # 146 of 1024 slots filled
    for step in range(6):
        q1 = (torch.randn(B, H, 1, D, generator=gen) * 0.7).to(dtype).cuda()
        k1 = (torch.randn(B, KVH, 1, D, generator=gen) * 0.7).to(dtype).cuda()
        v1 = (torch.randn(B, KVH, 1, D, generator=gen) * 0.7).to(dtype).cuda()
        out_a, new_a = cascade_attention(q1, k1, v1, with_hint, 0, inv_freq)
        out_b, new_b = cascade_attention(q1, k1, v1, without, 0, inv_freq, replayable=True)
        torch.cuda.synchronize()
        assert torch.equal(out_a.view(torch.uint8), out_b.view(torch.uint8)), f"step {step}: out"
        assert torch.equal(new_a.view(torch.uint8), new_b.view(torch.uint8)), f"step {step}: new scores"
        for name in STATE:
            a, b = getattr(with_hint, name)[0], getattr(without, name)[0]
            assert torch.equal(a.view(torch.uint8) if a.dtype.is_floating_point else a,
                               b.view(torch.uint8) if b.dtype.is_floating_point else b), f"step {step}: {name}"
