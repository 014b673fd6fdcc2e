"""GPU parity of ckv_update (through the C ABI) against the CPU oracle: every state tensor must
be bit-identical after every call."""
import random

import pytest
import torch

from oracle.update import CASCADE_FUNCS, OracleCache

pytestmark = pytest.mark.gpu

STATE = ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask", "pos",
         "og_pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")


def make_pair(B, H, D, NS, W, C, dtype, func="pow2", eager=True):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    gpu = CascadingKVCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=H, dim=D,
                           max_seq_len=W * C, device="cuda:0", dtype=dtype, cascade_func=func, layers=1,
                           eager_fill=eager, verbose=False)
    cpu = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=H, dim=D, max_seq_len=W * C,
                      dtype=dtype, cascade_func=func, eager_fill=eager)
    return gpu, cpu


def assert_same_state(gpu, cpu, ctx=""):
    torch.cuda.synchronize()
    for name in STATE:
        g = getattr(gpu, name)[0].cpu()
        c = getattr(cpu, name)
        if g.dtype.is_floating_point:  # compare bit patterns so that NaN payloads and -0.0 count
            same = torch.equal(g.view(torch.int16 if g.element_size() == 2 else torch.int32),
                               c.view(torch.int16 if c.element_size() == 2 else torch.int32))
        else:
            same = torch.equal(g, c)
        if not same:
            bad = (g != c).nonzero()[:5].tolist()
            raise AssertionError(f"{name} differs {ctx}; first mismatches at {bad}")
    assert int(gpu.seen_tokens_by_layer[0]) == int(cpu.seen_tokens)


def run_stream(gpu, cpu, n, chunker, gen, dtype, score_mode, transposed=False):
    B, H, D = cpu.max_batch_size, cpu.heads, cpu.dim
    done = 0
    call = 0
    while done < n:
        q = min(chunker(), n - done)
        if transposed:  # the layout a projection output has: (B, q, H, D) viewed as (B, H, q, D)
            k = torch.randn(B, q, H, D, generator=gen).to(dtype).transpose(1, 2)
            v = torch.randn(B, q, H, D, generator=gen).to(dtype).transpose(1, 2)
        else:
            k = torch.randn(B, H, q, D, generator=gen).to(dtype)
            v = torch.randn(B, H, q, D, generator=gen).to(dtype)
        if score_mode == "zero":
            s = None
        elif score_mode == "ties":
            s = (torch.randint(0, 4, (B, H, q), generator=gen).float() / 8).to(dtype)
        else:
            s = (torch.rand(B, H, q, generator=gen) * 1e-6).to(dtype)
        kg, vg = k.to("cuda:0"), v.to("cuda:0")
        if transposed:
            kg = k.transpose(1, 2).contiguous().to("cuda:0").transpose(1, 2)
            vg = v.transpose(1, 2).contiguous().to("cuda:0").transpose(1, 2)
        gpu.update(kg, vg, 0, None if s is None else s.to("cuda:0"))
        cpu.update(k, v, s)
        assert_same_state(gpu, cpu, f"after call {call} (q={q}, done={done})")
        done += q
        call += 1


@pytest.mark.parametrize("seed", range(12))
def test_random_small_streams(seed):
    rng = random.Random(seed)
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    B, H = rng.choice([1, 2]), rng.choice([1, 3])
    D = rng.choice([8, 16, 64, 128])
    NS = rng.choice([0, 1, 4, 7])
    W = rng.choice([1, 2, 3, 4, 8, 16])
    C = rng.choice([1, 2, 3, 4, 5, 8])
    func = rng.choice(CASCADE_FUNCS)
    eager = rng.random() < 0.5
    gpu, cpu = make_pair(B, H, D, NS, W, C, dtype, func, eager)
    gen = torch.Generator().manual_seed(seed)
    n = rng.randint(1, 30 * W + 20)
    mode = rng.choice(["zero", "ties", "rand"])
    print(f"seed={seed} dtype={dtype} B={B} H={H} D={D} NS={NS} W={W} C={C} {func} eager={eager} n={n} {mode}",
          flush=True)
    run_stream(gpu, cpu, n, lambda: rng.randint(1, 3 * W + 5), gen, dtype, mode)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_config1_shape(dtype):
    """B=1, 8 kv heads, D=128, sink 4, window 512 in C=4 cascades, 4096 tokens in chunks of 256."""
    gpu, cpu = make_pair(1, 8, 128, 4, 128, 4, dtype)
    gen = torch.Generator().manual_seed(1)
    run_stream(gpu, cpu, 4096, lambda: 256, gen, dtype, "ties", transposed=True)


def test_chunk_longer_than_cascade_window():
    """q > W: tokens cross a whole cascade inside one call (the Qwen2-shaped configuration)."""
    gpu, cpu = make_pair(2, 2, 64, 8, 32, 8, torch.bfloat16)
    gen = torch.Generator().manual_seed(5)
    run_stream(gpu, cpu, 2000, lambda: 100, gen, torch.bfloat16, "ties")
    gpu, cpu = make_pair(1, 2, 64, 8, 16, 4, torch.bfloat16, eager=False)
    run_stream(gpu, cpu, 1500, lambda: 500, gen, torch.bfloat16, "rand")


@pytest.mark.parametrize("B,H,D,NS,W,C,dtype,func,eager,mode", [
    # 32 or more (batch, kv head) units: plan, row moves and position ids of a unit in one launch
    (8, 4, 128, 4, 8, 4, torch.bfloat16, "pow2", True, "ties"),
    (11, 3, 64, 7, 5, 3, torch.float32, "pow2", False, "rand"),     # odd window: position ids one by one
    (16, 2, 128, 0, 16, 8, torch.float16, "pow2", False, "ties"),   # no sinks
    (4, 8, 256, 2, 4, 16, torch.float32, "pow2", True, "zero"),     # 16 cascades, 64 row pieces: that kernel's limits
    (4, 8, 16, 3, 4, 20, torch.bfloat16, "pow2", False, "ties"),    # more cascades than that: plan and apply launches
    (4, 8, 5, 2, 4, 3, torch.float32, "pow2", True, "ties"),        # 20-byte rows: plan launch, elementwise apply kernel
    (2, 4, 128, 4, 8, 4, torch.bfloat16, "pow2", True, "ties"),     # few units: plan and apply launches
] + [(8, 4, 32, 4, 6, 4, torch.bfloat16, f, e, "ties") for f in CASCADE_FUNCS for e in (True, False)])
def test_single_token_calls(B, H, D, NS, W, C, dtype, func, eager, mode):
    """One token per call (the decode step): plan, row moves and position ids of a unit in one launch where the
    layout allows it and the units are many, the two-launch path elsewhere; every acceptance schedule, with and
    without eager fill."""
    gpu, cpu = make_pair(B, H, D, NS, W, C, dtype, func, eager)
    gen = torch.Generator().manual_seed(6)
    run_stream(gpu, cpu, NS + 3 * W * C + 40, lambda: 1, gen, dtype, mode)


def test_call_larger_than_one_launch():
    """More tokens than one planning launch holds in LDS: the call is split internally."""
    gpu, cpu = make_pair(1, 2, 16, 4, 64, 4, torch.float32, eager=False)
    gen = torch.Generator().manual_seed(7)
    run_stream(gpu, cpu, 12000, lambda: 6000, gen, torch.float32, "ties")


def test_unaligned_layout_takes_elementwise_path():
    gpu, cpu = make_pair(1, 2, 5, 2, 4, 3, torch.float32)  # 20-byte rows
    gen = torch.Generator().manual_seed(8)
    run_stream(gpu, cpu, 200, lambda: 7, gen, torch.float32, "ties")
    gpu, cpu = make_pair(1, 2, 3, 2, 4, 3, torch.float16)   # 6-byte rows
    run_stream(gpu, cpu, 200, lambda: 9, gen, torch.float16, "rand")


def test_config2_shape_prefill_chunks():
    """B=2, 8 kv heads, D=128, sink 64, 16384 slots in C=8 cascades, 2048-token chunks."""
    gpu, cpu = make_pair(2, 8, 128, 64, 2048, 8, torch.bfloat16)
    gen = torch.Generator().manual_seed(2)
    run_stream(gpu, cpu, 2048 * 12, lambda: 2048, gen, torch.bfloat16, "ties", transposed=True)


def test_reference_preconditions_and_errors():
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    with pytest.raises(ValueError):
        CascadingKVCache(window_length=3, max_seq_len=8, layers=1, device="cuda:0", verbose=False)
    with pytest.raises(ValueError):
        CascadingKVCache(window_length=[4], max_seq_len=8, layers=1, device="cuda:0", verbose=False)
    with pytest.raises(ValueError):
        CascadingKVCache(window_length=4, max_seq_len=8, layers=1, cascade_func="nope", device="cuda:0",
                         verbose=False)
    c = CascadingKVCache(window_length=4, num_sink_tokens=2, max_batch_size=1, heads=1, dim=8, max_seq_len=8,
                         device="cuda:0", dtype=torch.float32, layers=1, verbose=False)
    with pytest.raises(_abi.CkvError):  # CPU tensors never fall back
        c.update(torch.zeros(1, 1, 2, 8), torch.zeros(1, 1, 2, 8), 0)
    with pytest.raises(TypeError):
        c.update(torch.zeros(1, 1, 2, 8, device="cuda:0", dtype=torch.float16),
                 torch.zeros(1, 1, 2, 8, device="cuda:0", dtype=torch.float16), 0,
                 torch.zeros(1, 1, 2, device="cuda:0", dtype=torch.float16))


def test_token_counter_by_table_and_by_device_counter():
    """An update reads the tokens seen so far from a constant table the host indexes, and the device counter
    ``seen_tokens_by_layer`` is brought up to date when it is read; past the end of the table (made tiny here) the
    update reads and advances the device counter itself.  Either way the original token indices (og_pos) and every
    other state tensor equal the oracle's."""
    from cascading_kv_cache_amd import cascading_cache as cc

    dtype = torch.float32
    gpu, cpu = make_pair(2, 2, 16, 2, 8, 2, dtype)
    gen = torch.Generator().manual_seed(5)

    def feed(q):
        k = torch.randn(2, 2, q, 16, generator=gen)
        v = torch.randn(2, 2, q, 16, generator=gen)
        s = (torch.rand(2, 2, q, generator=gen) * 1e-6)
        gpu.update_state(k.cuda(), v.cuda(), 0, s.cuda())
        cpu.update(k, v, s)

    for q in (3, 1, 5, 1, 1):          # nobody looks at the device counter in between
        feed(q)
    assert gpu._seen_pending == [11] and int(gpu._seen_dev[0]) == 0
    assert int(gpu.seen_tokens_by_layer[0]) == 11 and gpu._seen_pending == [0]
    assert_same_state(gpu, cpu, "by the table")

    key = ("cuda", 0)
    full = cc._COUNTER_TABLES[key]
    try:
        cc._COUNTER_TABLES[key] = full[:13]        # tokens 11 and 12 still come from the table, later ones do not
        for q in (1, 1, 4, 1, 7):
            feed(q)
        assert gpu._seen_pending == [0] and int(gpu._seen_dev[0]) == 25
        assert_same_state(gpu, cpu, "by the device counter")
    finally:
        cc._COUNTER_TABLES[key] = full
    feed(2)
    assert gpu._seen_pending == [2]
    assert_same_state(gpu, cpu, "back on the table")
