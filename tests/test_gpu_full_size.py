"""The benchmark configurations at their real shapes.  The oracle's attention would take minutes here, so
attention is checked through size-independent properties and sampled rows against float64 dense attention;
the cache update is cheap enough on the CPU to be compared bit for bit at full size.
Config 2: B=2, 32q/8kv heads, head_dim 128, 64 sinks + 8 x 2048 slots, 2048-token chunks; config 3: B=16,
64 sinks + 4 x 8192 slots, one token; config 4 (one layer of it): B=1, 64 sinks + 8 x 8192 slots, 4096-token
chunks; config 5 (one layer): B=4, 28q/4kv heads, 64 sinks + 16 x 2048 slots, 4096-token chunks (longer than
a cascade window)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

STATE = ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask", "pos", "og_pos",
         "sink_pos", "stored_tokens", "start_indices", "stored_sinks")


def make_cache(B, KVH, D, NS, S, C, dtype):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    return CascadingKVCache(window_length=S // C, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D, max_seq_len=S,
                            device="cuda:0", dtype=dtype, cascade_func="pow2", head_reduction="mean", layers=1,
                            eager_fill=True, verbose=False)


def chunk(B, H, KVH, Q, D, gen, dtype):
    q = (torch.randn(B, H, Q, D, generator=gen) * 0.3).to(dtype).cuda()
    k = (torch.randn(B, KVH, Q, D, generator=gen) * 0.3).to(dtype).cuda()
    v = (torch.randn(B, KVH, Q, D, generator=gen) * 0.3).to(dtype).cuda()
    return q, k, v


def snapshot(cache):
    return {n: getattr(cache, n)[0].clone() for n in STATE}, cache._seen_host[0], cache.seen_tokens_by_layer.clone()


def restore(cache, snap):
    tensors, seen_host, seen = snap
    for n, t in tensors.items():
        getattr(cache, n)[0].copy_(t)
    cache._seen_host[0] = seen_host
    cache.seen_tokens_by_layer.copy_(seen)


CFG2 = dict(B=2, H=32, KVH=8, D=128, NS=64, S=16384, C=8, Q=2048, fill=10, fill_q=2048, theta=5e5)
CFG4 = dict(B=1, H=32, KVH=8, D=128, NS=64, S=65536, C=8, Q=4096, fill=18, fill_q=4096, theta=5e5)
CFG5 = dict(B=4, H=28, KVH=4, D=128, NS=64, S=32768, C=16, Q=4096, fill=10, fill_q=4096, theta=1e6)


@pytest.mark.parametrize("cfg", [
    CFG2,                                                                               # cache full and evicting
    dict(B=16, H=32, KVH=8, D=128, NS=64, S=32768, C=4, Q=1, fill=3, fill_q=2048, theta=5e5),   # decode, cache partly filled
    CFG4, CFG5,
    dict(CFG4, Q=1), dict(CFG5, Q=1),                                                   # single-token steps on the same caches
], ids=["cfg2", "cfg3-partly-filled", "cfg4", "cfg5", "cfg4-decode", "cfg5-decode"])
def test_full_size_properties(cfg):
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    dtype = torch.bfloat16
    B, H, KVH, D, Q = cfg["B"], cfg["H"], cfg["KVH"], cfg["D"], cfg["Q"]
    cache = make_cache(B, KVH, D, cfg["NS"], cfg["S"], cfg["C"], dtype)
    inv_freq = default_inv_freq(D, cfg["theta"], "cuda:0")
    gen = torch.Generator().manual_seed(7)
    for _ in range(cfg["fill"]):   # chunks through the real path
        cascade_attention(*chunk(B, H, KVH, cfg["fill_q"], D, gen, dtype), cache, 0, inv_freq)
    q, k, v = chunk(B, H, KVH, Q, D, gen, dtype)
    snap = snapshot(cache)

    # 1. determinism: the same call from the same state gives the same bits everywhere
    out1, new1 = cascade_attention(q, k, v, cache, 0, inv_freq)
    after1 = snapshot(cache)
    restore(cache, snap)
    out2, new2 = cascade_attention(q, k, v, cache, 0, inv_freq)
    after2 = snapshot(cache)
    assert torch.equal(out1, out2) and torch.equal(new1, new2)
    for n in STATE:
        assert torch.equal(after1[0][n], after2[0][n]), n
    assert torch.isfinite(out1.float()).all()

    # 2. the rows of P sum to one: with every value row equal to one vector c, every output row is c
    restore(cache, snap)
    c = torch.linspace(-1.0, 1.0, D).to(dtype).cuda()
    cache.value_cache[0][:] = c
    cache.sink_values[0][:] = c
    out_c, _ = cascade_attention(q, k, c.expand(B, KVH, Q, D).contiguous(), cache, 0, inv_freq, update_cache=False)
    err = (out_c.float() - c.float()).abs().max().item()
    assert err <= 1.5e-2, f"softmax rows do not sum to one: max deviation {err:.3e}"

    # 3. linear in V: out(V) + out(V') = out(V + V') up to the rounding of three bf16 results
    restore(cache, snap)
    out_a, _ = cascade_attention(q, k, v, cache, 0, inv_freq, update_cache=False)
    half = snapshot(cache)
    restore(cache, snap)
    cache.value_cache[0].mul_(0.5)
    cache.sink_values[0].mul_(0.5)
    out_h, _ = cascade_attention(q, k, (v * 0.5), cache, 0, inv_freq, update_cache=False)
    assert (out_a.float() - 2 * out_h.float()).abs().max().item() <= 1e-2  # exact scaling by a power of two, up to P rounding

    # 4. the score EMA after the call does not depend on V at all
    assert torch.equal(half[0]["score_cache"], snapshot(cache)[0]["score_cache"])


def _rope64(x, pos, theta=5e5):
    """Textbook rotary embedding in float64 with complex numbers: pairs (x[d], x[d + D/2])."""
    D = x.size(-1)
    xd = x.double()
    z = torch.complex(xd[..., : D // 2], xd[..., D // 2:])
    freq = theta ** (-torch.arange(0, D, 2, dtype=torch.float64) / D)
    ang = pos.double()[..., None] * freq
    z = z * torch.polar(torch.ones_like(ang), ang)
    return torch.cat((z.real, z.imag), dim=-1)


@pytest.mark.parametrize("cfg", [
    CFG2,
    dict(B=16, H=32, KVH=8, D=128, NS=64, S=32768, C=4, Q=1, fill=17, fill_q=2048, theta=5e5),   # decode with the cache full
    CFG4, CFG5, dict(CFG4, Q=1), dict(CFG5, Q=1),
], ids=["cfg2", "cfg3", "cfg4", "cfg5", "cfg4-decode", "cfg5-decode"])
def test_full_size_sampled_rows_against_dense_attention(cfg):
    """At the benchmark sizes the whole oracle takes minutes, a few rows of it do not: for sampled
    (batch, head, query) rows, softmax(q K^T / sqrt(D)) V over exactly the visible keys in float64, with
    complex-number RoPE at the cache's position ids, against the library's output (2e-2 abs, bf16)."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, chunk_positions, default_inv_freq

    dtype = torch.bfloat16
    B, H, KVH, D, Q, NS = cfg["B"], cfg["H"], cfg["KVH"], cfg["D"], cfg["Q"], cfg["NS"]
    G = H // KVH
    cache = make_cache(B, KVH, D, NS, cfg["S"], cfg["C"], dtype)
    theta = cfg["theta"]
    inv_freq = default_inv_freq(D, theta, "cuda:0")
    gen = torch.Generator().manual_seed(9)
    for _ in range(cfg["fill"]):
        cascade_attention(*chunk(B, H, KVH, cfg["fill_q"], D, gen, dtype), cache, 0, inv_freq)
    q, k, v = chunk(B, H, KVH, Q, D, gen, dtype)
    # what the call will see: the state before it
    vals = [t.clone() for t in cache.get_vals(0)]
    sink_k, sink_v, sink_pos, sink_mask, ck, cv, key_pos, key_mask, _ = vals
    q_pos = chunk_positions(cache, 0, Q).cpu().view(-1)
    out, _ = cascade_attention(q, k, v, cache, 0, inv_freq, update_cache=False)
    torch.cuda.synchronize()
    sv, cvalid = (~sink_mask[0, 0]).cpu(), (~key_mask[0, 0]).cpu()
    assert int(cvalid.sum()) == cfg["S"], "the cache should be full at this point"
    sink_pos, key_pos = sink_pos[0].cpu(), key_pos[0].cpu()
    rows = [(0, 0, 0), (B - 1, H - 1, Q - 1), (B // 2, 5, Q // 2), (0, 17, min(Q - 1, 63)), (B - 1, 30 % H, min(Q - 1, 64)),
            (0, 9, max(0, Q - 700))]
    worst = 0.0
    for b, h, m in rows:
        kvh = h // G
        keys = torch.cat((_rope64(sink_k[b, kvh].cpu()[sv], sink_pos[sv], theta),
                          _rope64(ck[b, kvh].cpu()[cvalid], key_pos[cvalid], theta),
                          _rope64(k[b, kvh, : m + 1].cpu(), q_pos[: m + 1], theta)), dim=0)
        valv = torch.cat((sink_v[b, kvh].cpu()[sv], cv[b, kvh].cpu()[cvalid], v[b, kvh, : m + 1].cpu()), dim=0).double()
        qr = _rope64(q[b, h, m].cpu(), q_pos[m], theta)
        p = torch.softmax(keys @ qr / (D ** 0.5), dim=0)
        want = p @ valv
        worst = max(worst, (out[b, h, m].double().cpu() - want).abs().max().item())
    assert worst <= 2e-2, f"sampled rows differ from dense attention by {worst:.3e}"


@pytest.mark.parametrize("cfg", [
    dict(B=1, KVH=8, D=128, NS=64, W=8192, C=8, q=4096, calls=20),      # config 4: 81920 tokens through 65536 slots
    dict(B=4, KVH=4, D=128, NS=64, W=2048, C=16, q=4096, calls=12),     # config 5: calls longer than a cascade window
], ids=["cfg4", "cfg5"])
def test_update_bit_exact_at_benchmark_shapes(cfg):
    """ckv_update against the serial oracle at the cache shapes of configs 4 and 5, for enough calls that every
    cascade is full and evicting: every state tensor bit-identical after every call (tie-heavy scores)."""
    from test_gpu_update import make_pair, run_stream

    dtype = torch.bfloat16
    gpu, cpu = make_pair(cfg["B"], cfg["KVH"], cfg["D"], cfg["NS"], cfg["W"], cfg["C"], dtype)
    gen = torch.Generator().manual_seed(41)
    run_stream(gpu, cpu, cfg["q"] * cfg["calls"], lambda: cfg["q"], gen, dtype, "ties", transposed=True)
    assert not bool(cpu.mask.any()) and int(cpu.start_indices[..., -1].sum()) > 0, "the last cascade must have evicted"


def test_config3_consecutive_decode_steps_update_bit_exact():
    """Config 3 at full size: B=16, 8 kv heads, 64 sinks + 4 x 8192 slots, cache full.  Eight single-token steps in a
    row through the real path (attention, score EMA, update); after every step the whole cache state must equal
    the oracle's update run on the same scores, bit for bit."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq
    from parity_helpers import STATE, bits, push_state
    from test_gpu_update import make_pair

    dtype = torch.bfloat16
    B, H, KVH, D, NS, W, C = 16, 32, 8, 128, 64, 8192, 4
    gpu, cpu = make_pair(B, KVH, D, NS, W, C, dtype)
    gen = torch.Generator().manual_seed(43)
    for _ in range(5):  # 40960 tokens through the oracle alone: cache full, every cascade evicting
        n = 8192
        k = torch.randn(B, KVH, n, D, generator=gen).to(dtype)
        v = torch.randn(B, KVH, n, D, generator=gen).to(dtype)
        cpu.update(k, v, (torch.rand(B, KVH, n, generator=gen) * 1e-6).to(dtype))
    del k, v
    push_state(gpu, cpu)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    for step in range(8):
        q = torch.randn(B, H, 1, D, generator=gen).to(dtype)
        k = torch.randn(B, KVH, 1, D, generator=gen).to(dtype)
        v = torch.randn(B, KVH, 1, D, generator=gen).to(dtype)
        out, new_g = cascade_attention(q.cuda(), k.cuda(), v.cuda(), gpu, 0, inv_freq, update_cache=False)
        assert torch.isfinite(out.float()).all()
        cpu.score_cache.copy_(gpu.score_cache[0])          # the update's score inputs are the library's own
        gpu.update(k.cuda(), v.cuda(), 0, score_states=new_g)
        cpu.update(k, v, new_g.cpu())
        torch.cuda.synchronize()
        heavy = step in (0, 3, 7)                          # the 1 GiB K and V caches are pulled back on these steps
        for name in STATE:
            if name in ("key_cache", "value_cache") and not heavy:
                continue
            g, w = bits(getattr(gpu, name)[0].cpu()), bits(getattr(cpu, name))
            assert torch.equal(g, w), f"step {step}: {name} differs from the oracle"
        assert int(gpu.seen_tokens_by_layer[0]) == int(cpu.seen_tokens)


def test_config3_all_1024_decode_steps():
    """Config 3 as it is written: the cache pre-filled full, then 1024 single-token steps in a row through the real
    path (attention, score EMA, update).  The oracle's update follows with the library's own scores; the trackers are
    compared after every step, every other state tensor but K and V every 64 steps, K and V at the end: bit for
    bit.  Outputs stay finite and the position ids a permutation throughout."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq
    from parity_helpers import STATE, bits, push_state
    from test_gpu_update import make_pair

    dtype = torch.bfloat16
    B, H, KVH, D, NS, W, C = 16, 32, 8, 128, 64, 8192, 4
    gpu, cpu = make_pair(B, KVH, D, NS, W, C, dtype)
    gen = torch.Generator().manual_seed(47)
    for _ in range(5):  # 40960 tokens through the oracle alone: cache full, every cascade evicting
        n = 8192
        k = torch.randn(B, KVH, n, D, generator=gen).to(dtype)
        v = torch.randn(B, KVH, n, D, generator=gen).to(dtype)
        cpu.update(k, v, (torch.rand(B, KVH, n, generator=gen) * 1e-6).to(dtype))
    del k, v
    push_state(gpu, cpu)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    qs = torch.randn(8, B, H, 1, D, generator=gen).to(dtype).cuda()
    ks = torch.randn(8, B, KVH, 1, D, generator=gen).to(dtype)
    vs = torch.randn(8, B, KVH, 1, D, generator=gen).to(dtype)
    ks_d, vs_d = ks.cuda(), vs.cuda()
    light = ("stored_tokens", "start_indices", "stored_sinks")
    for step in range(1024):
        i = step % 8
        out, new_g = cascade_attention(qs[i], ks_d[i], vs_d[i], gpu, 0, inv_freq, update_cache=False)
        cpu.score_cache.copy_(gpu.score_cache[0])          # the update's score inputs are the library's own
        gpu.update(ks_d[i], vs_d[i], 0, score_states=new_g)
        cpu.update(ks[i], vs[i], new_g.cpu())
        last = step == 1023
        names = STATE if last else (tuple(n for n in STATE if n not in ("key_cache", "value_cache")) if step % 64 == 63 else light)
        for name in names:
            g, w = bits(getattr(gpu, name)[0].cpu()), bits(getattr(cpu, name))
            assert torch.equal(g, w), f"step {step}: {name} differs from the oracle"
        if step % 64 == 63 or last:
            assert bool(torch.isfinite(out.float()).all()), f"step {step}: output"
            row = gpu.pos[0][0, 0].sort().values
            assert torch.equal(row, torch.arange(W * C, device="cuda:0")), f"step {step}: position ids"
    assert int(gpu.seen_tokens_by_layer[0]) == int(cpu.seen_tokens) == 5 * 8192 + 1024
