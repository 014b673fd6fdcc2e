"""Single-token steps replayed from a HIP graph (DecodeStepGraph) against the same steps launched eagerly:
outputs, new scores and every state tensor bit-identical after every step.  The graph is replayed many times
with eager work of the program and synchronisations in between, and every replay is checked."""
import pytest
import torch

from parity_helpers import STATE, bits

pytestmark = pytest.mark.gpu


def make_cache(B, KVH, D, NS, W, C, dtype, eager):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    return CascadingKVCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D,
                            max_seq_len=W * C, device="cuda:0", dtype=dtype, head_reduction="max", layers=2,
                            eager_fill=eager, verbose=False)


@pytest.mark.parametrize("eager_fill,B,H,KVH,chunks", [(True, 1, 8, 2, 5), (False, 2, 14, 2, 5), (True, 1, 8, 2, 4), (True, 2, 8, 2, 1)])
def test_graph_replayed_steps_equal_eager_steps(eager_fill, B, H, KVH, chunks):
    from cascading_kv_cache_amd.cascade_attention import DecodeStepGraph, cascade_attention, default_inv_freq

    dtype, D, NS, W, C = torch.bfloat16, 128, 4, 64, 4
    ref, rep = make_cache(B, KVH, D, NS, W, C, dtype, eager_fill), make_cache(B, KVH, D, NS, W, C, dtype, eager_fill)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(23)
    L = 1  # a layer other than the first: the graph must address that layer's state
    # 5 chunks: past the window, the cascades evict; 4: the cache fills up during the replayed steps; 1: it stays
    # mostly empty, and the position ids and the filled part differ from step to step
    for _ in range(chunks):
        q = (torch.randn(B, H, 60, D, generator=gen) * 0.7).to(dtype).cuda()
        k = (torch.randn(B, KVH, 60, D, generator=gen) * 0.7).to(dtype).cuda()
        v = (torch.randn(B, KVH, 60, D, generator=gen) * 0.7).to(dtype).cuda()
        for c in (ref, rep):
            cascade_attention(q, k, v, c, L, inv_freq)
    graph = DecodeStepGraph(rep, L, inv_freq, H)
    scratch = torch.zeros(1 << 16, device="cuda:0")
    for step in range(24):
        q = (torch.randn(B, H, 1, D, generator=gen) * 0.7).to(dtype).cuda()
        k = (torch.randn(B, KVH, 1, D, generator=gen) * 0.7).to(dtype).cuda()
        v = (torch.randn(B, KVH, 1, D, generator=gen) * 0.7).to(dtype).cuda()
        out_e, new_e = cascade_attention(q, k, v, ref, L, inv_freq)
        out_g, new_g = graph.step(q, k, v)
        # eager work of the program and a synchronisation between two replays
        scratch.add_(1.0).mul_(0.5)
        torch.cuda.synchronize()
        assert torch.equal(bits(out_g), bits(out_e)), f"step {step}: out"
        assert torch.equal(bits(new_g), bits(new_e)), f"step {step}: new scores"
        for name in STATE:
            assert torch.equal(bits(getattr(rep, name)[L]), bits(getattr(ref, name)[L])), f"step {step}: {name}"
        assert torch.equal(rep.seen_tokens_by_layer, ref.seen_tokens_by_layer) and rep._seen_host == ref._seen_host
    assert graph.graph is not None  # steps 2.. were replays


def test_graph_refuses_a_cache_whose_state_moved():
    from cascading_kv_cache_amd import _abi
    from cascading_kv_cache_amd.cascade_attention import DecodeStepGraph, cascade_attention, default_inv_freq

    dtype, B, H, KVH, D = torch.bfloat16, 1, 4, 2, 128
    cache = make_cache(B, KVH, D, 4, 32, 2, dtype, True)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    graph = DecodeStepGraph(cache, 0, inv_freq, H)
    q = torch.zeros(B, H, 1, D, dtype=dtype, device="cuda:0")
    k = torch.zeros(B, KVH, 1, D, dtype=dtype, device="cuda:0")
    with pytest.raises(_abi.CkvError):  # no token in the cache yet: the sink shift would still change
        graph.step(q, k, k)
    big = torch.zeros(B, H, 40, D, dtype=dtype, device="cuda:0")
    cascade_attention(big, big[:, :KVH], big[:, :KVH], cache, 0, inv_freq)
    for _ in range(3):
        graph.step(q, k, k)
    cache.score_cache[0] = cache.score_cache[0].clone()
    with pytest.raises(_abi.CkvError):
        graph.step(q, k, k)


def test_graph_survives_a_reset_of_its_cache():
    """A step recorded on a full, eagerly filled cache; then ``reset()`` (which zeroes every state tensor in
    place, so no address changes) and a partial refill: later steps must equal eager steps bit for bit — the
    position ids of the token must come from the cache as it is now, not from the time of the recording."""
    from cascading_kv_cache_amd.cascade_attention import DecodeStepGraph, cascade_attention, default_inv_freq

    dtype, B, H, KVH, D, NS, W, C = torch.bfloat16, 1, 8, 2, 128, 4, 32, 2
    ref, rep = make_cache(B, KVH, D, NS, W, C, dtype, True), make_cache(B, KVH, D, NS, W, C, dtype, True)
    inv_freq = default_inv_freq(D, 5e5, "cuda:0")
    gen = torch.Generator().manual_seed(5)

    def chunk(n):
        q = (torch.randn(B, H, n, D, generator=gen) * 0.7).to(dtype).cuda()
        k = (torch.randn(B, KVH, n, D, generator=gen) * 0.7).to(dtype).cuda()
        v = (torch.randn(B, KVH, n, D, generator=gen) * 0.7).to(dtype).cuda()
        return q, k, v

    def both_step(graph, what):
        q, k, v = chunk(1)
        out_e, new_e = cascade_attention(q, k, v, ref, 0, inv_freq)
        out_g, new_g = graph.step(q, k, v)
        torch.cuda.synchronize()
        assert torch.equal(bits(out_g), bits(out_e)), f"{what}: out"
        assert torch.equal(bits(new_g), bits(new_e)), f"{what}: new scores"
        for name in STATE:
            assert torch.equal(bits(getattr(rep, name)[0]), bits(getattr(ref, name)[0])), f"{what}: {name}"

    q, k, v = chunk(W * C + NS + 10)       # more than the cache holds: full and evicting
    for c in (ref, rep):
        cascade_attention(q, k, v, c, 0, inv_freq)
    graph = DecodeStepGraph(rep, 0, inv_freq, H)
    for step in range(4):
        both_step(graph, f"full cache, step {step}")
    assert graph.graph is not None
    for c in (ref, rep):
        c.reset(verbose=False)
    q, k, v = chunk(NS + 9)                # past the sinks, far from full
    for c in (ref, rep):
        cascade_attention(q, k, v, c, 0, inv_freq)
    for step in range(6):
        both_step(graph, f"after reset, step {step}")
    assert graph.graph is not None          # recorded again after the reset
