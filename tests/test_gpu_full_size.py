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
    dict(B=2, H=32, KVH=8, D=128, NS=64, S=16384, C=8, Q=2048, fill=10),
    dict(B=16, H=32, KVH=8, D=128, NS=64, S=32768, C=4, Q=1, fill=17),     # decode with the cache full
])
def test_full_size_sampled_rows_against_dense_attention(cfg):
    """At the benchmark sizes the whole oracle takes minutes, a few rows of it do not: for sampled
    (batch, head, query) rows, softmax(q K^T / sqrt(D)) V over exactly the visible keys in float64, with
    complex-number RoPE at the cache's position ids, against the library's output (2e-2 abs, bf16)."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, chunk_positions, default_inv_freq

    dtype = torch.bfloat16
    B, H, KVH, D, Q, NS = cfg["B"], cfg["H"], cfg["KVH"], cfg["D"], cfg["Q"], cfg["NS"]
    G = H // KVH
    cache = make_cache(B, KVH, D, NS, cfg["S"], cfg["C"], dtype)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(9)
    for _ in range(cfg["fill"]):
        cascade_attention(*chunk(B, H, KVH, 2048, D, gen, dtype), cache, 0, inv_freq)
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
    rows = [(0, 0, 0), (B - 1, H - 1, Q - 1), (B // 2, 5, Q // 2), (0, 17, min(Q - 1, 63)), (B - 1, 30, min(Q - 1, 64)),
            (0, 9, max(0, Q - 700))]
    worst = 0.0
    for b, h, m in rows:
        kvh = h // G
        keys = torch.cat((_rope64(sink_k[b, kvh].cpu()[sv], sink_pos[sv]),
                          _rope64(ck[b, kvh].cpu()[cvalid], key_pos[cvalid]),
                          _rope64(k[b, kvh, : m + 1].cpu(), q_pos[: m + 1])), dim=0)
        valv = torch.cat((sink_v[b, kvh].cpu()[sv], cv[b, kvh].cpu()[cvalid], v[b, kvh, : m + 1].cpu()), dim=0).double()
        qr = _rope64(q[b, h, m].cpu(), q_pos[m])
        p = torch.softmax(keys @ qr / (D ** 0.5), dim=0)
        want = p @ valv
        worst = max(worst, (out[b, h, m].double().cpu() - want).abs().max().item())
    assert worst <= 2e-2, f"sampled rows differ from dense attention by {worst:.3e}"
