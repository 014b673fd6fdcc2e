"""Size-independent properties at the full benchmark sizes (no oracle: the CPU restatement would take
minutes here).  Config 2: B=2, 32q/8kv heads, head_dim 128, 64 sinks + 8 x 2048 slots, 2048-token
chunks; config 3: B=16, 64 sinks + 4 x 8192 slots, one token."""
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


@pytest.mark.parametrize("cfg", [
    dict(B=2, H=32, KVH=8, D=128, NS=64, S=16384, C=8, Q=2048, fill=10),   # chunked prefill, cache full and evicting
    dict(B=16, H=32, KVH=8, D=128, NS=64, S=32768, C=4, Q=1, fill=3),      # decode, cache partly filled
])
def test_full_size_properties(cfg):
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq

    dtype = torch.bfloat16
    B, H, KVH, D, Q = cfg["B"], cfg["H"], cfg["KVH"], cfg["D"], cfg["Q"]
    cache = make_cache(B, KVH, D, cfg["NS"], cfg["S"], cfg["C"], dtype)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(7)
    for _ in range(cfg["fill"]):   # 2048-token chunks through the real path
        cascade_attention(*chunk(B, H, KVH, 2048, D, gen, dtype), cache, 0, inv_freq)
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
