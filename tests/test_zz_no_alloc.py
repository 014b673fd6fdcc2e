"""ckv_update_static (the entry point that allocates nothing: its scratch is a fixed array inside the
library) against ckv_update (scratch from the caller), through the C ABI: every state tensor bit-identical
after two calls in a row on the same device, the second with a smaller input, so the shared scratch still
holds what the first call left there."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu

STATE = ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask", "pos",
         "og_pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")


def make_cache(B, KVH, D, NS, W, Cn, dtype):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    return CascadingKVCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D,
                            max_seq_len=W * Cn, device="cuda:0", dtype=dtype, layers=1, eager_fill=False,
                            verbose=False)


def describe(cache, k, v, s):
    from cascading_kv_cache_amd import _abi

    return _abi.fill_update_args(k, v, s, cache.sink_keys[0], cache.sink_values[0], cache.sink_mask[0],
                                 cache.sink_pos[0], cache.key_cache[0], cache.value_cache[0], cache.score_cache[0],
                                 cache.mask[0], cache.pos[0], cache.og_pos[0], cache.do_cache_every_n[0],
                                 cache.stored_tokens[0], cache.start_indices[0], cache.stored_sinks[0],
                                 cache.num_sink_tokens, cache.window_length[0], cache.seen_tokens_by_layer[0],
                                 cache.max_seq_len[0], cache.eager_fill)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_update_matches_the_workspace_entry_point(dtype):
    from cascading_kv_cache_amd import _abi

    lib = _abi.lib()
    B, KVH, D, NS, W, Cn = 2, 4, 128, 4, 64, 4
    ref, sta = make_cache(B, KVH, D, NS, W, Cn, dtype), make_cache(B, KVH, D, NS, W, Cn, dtype)
    gen = torch.Generator().manual_seed(17)
    stream = torch.cuda.current_stream().cuda_stream
    # two fills, then the pair the task names: a large call and right after it a smaller one
    for call, q in enumerate((300, 300, 700, 90, 1)):
        k = torch.randn(B, KVH, q, D, generator=gen).to(dtype).cuda()
        v = torch.randn(B, KVH, q, D, generator=gen).to(dtype).cuda()
        s = (torch.randint(0, 6, (B, KVH, q), generator=gen).float() / 8).to(dtype).cuda()  # ties included
        a = describe(ref, k, v, s)
        need = lib.ckv_update_workspace_bytes(a.N, a.H, a.K, a.max_seq_len, a.cascades)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda:0")
        a.workspace, a.workspace_bytes = ws.data_ptr(), need
        _abi.check(lib.ckv_update(C.byref(a), C.c_void_p(stream)), "ckv_update")
        b = describe(sta, k, v, s)  # no workspace: the entry point brings its own
        assert b.workspace is None and b.workspace_bytes == 0
        _abi.check(lib.ckv_update_static(C.byref(b), C.c_void_p(stream)), "ckv_update_static")
        for c in (ref, sta):
            c.seen_tokens_by_layer[0] += q
            c._seen_host[0] += q
        torch.cuda.synchronize()
        for name in STATE:
            g, w = getattr(sta, name)[0], getattr(ref, name)[0]
            if g.dtype.is_floating_point:
                it = torch.int16 if g.element_size() == 2 else torch.int32
                g, w = g.view(it), w.view(it)
            assert torch.equal(g, w), f"call {call} (q={q}): {name} differs between the two entry points"
    assert int((~ref.mask[0]).sum()) > 0


def test_static_scratch_update_refuses_sizes_beyond_its_array():
    from cascading_kv_cache_amd import _abi

    lib = _abi.lib()
    limit = lib.ckv_update_static_scratch_bytes()
    assert limit == 32 << 20
    # 16 x 8 units of 131072 slots: the move chains alone need 64 MiB
    B, KVH, D, NS, W, Cn = 16, 8, 8, 4, 32768, 4
    assert lib.ckv_update_workspace_bytes(B, KVH, 1, W * Cn, Cn) > limit
    cache = make_cache(B, KVH, D, NS, W, Cn, torch.bfloat16)
    before = {n: getattr(cache, n)[0].clone() for n in STATE}
    k = torch.zeros(B, KVH, 1, D, dtype=torch.bfloat16, device="cuda:0")
    a = describe(cache, k, k.clone(), torch.zeros(B, KVH, 1, dtype=torch.bfloat16, device="cuda:0"))
    rc = lib.ckv_update_static(C.byref(a), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -8 and b"ckv_update_static" in lib.ckv_strerror(rc)
    torch.cuda.synchronize()
    for n in STATE:
        assert torch.equal(getattr(cache, n)[0], before[n]), f"{n} was touched by a refused call"


def test_static_scratch_update_recorded_into_a_graph():
    """The callers the entry point is for include code under HIP graph capture: after one ordinary call on the
    device (which looks the array's address and the device's limits up), the call is recorded, and every replay —
    with eager work and synchronisations of the program in between, fresh inputs copied into the recorded buffers —
    leaves the state bit-identical to ckv_update on a second cache."""
    from cascading_kv_cache_amd import _abi

    lib = _abi.lib()
    dtype = torch.bfloat16
    B, KVH, D, NS, W, Cn, q = 2, 2, 128, 4, 32, 4, 24
    ref, sta = make_cache(B, KVH, D, NS, W, Cn, dtype), make_cache(B, KVH, D, NS, W, Cn, dtype)
    gen = torch.Generator().manual_seed(29)
    k = torch.zeros(B, KVH, q, D, dtype=dtype, device="cuda:0")
    v, s = torch.zeros_like(k), torch.zeros(B, KVH, q, dtype=dtype, device="cuda:0")
    a, b = describe(ref, k, v, s), describe(sta, k, v, s)
    need = lib.ckv_update_workspace_bytes(a.N, a.H, a.K, a.max_seq_len, a.cascades)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda:0")
    a.workspace, a.workspace_bytes = ws.data_ptr(), need

    def fresh_inputs():
        k.copy_(torch.randn(B, KVH, q, D, generator=gen).to(dtype))
        v.copy_(torch.randn(B, KVH, q, D, generator=gen).to(dtype))
        s.copy_((torch.randint(0, 6, (B, KVH, q), generator=gen).float() / 8).to(dtype))

    def advance():
        for c in (ref, sta):
            c.seen_tokens_by_layer[0] += q
            c._seen_host[0] += q

    def same(what):
        torch.cuda.synchronize()
        for name in STATE:
            g, w = getattr(sta, name)[0], getattr(ref, name)[0]
            if g.dtype.is_floating_point:
                g, w = g.view(torch.int16), w.view(torch.int16)
            assert torch.equal(g, w), f"{what}: {name}"

    # the ordinary call that must come first on a device
    fresh_inputs()
    stream = torch.cuda.current_stream().cuda_stream
    _abi.check(lib.ckv_update(C.byref(a), C.c_void_p(stream)), "ckv_update")
    _abi.check(lib.ckv_update_static(C.byref(b), C.c_void_p(stream)), "ckv_update_static")
    advance()
    same("eager call")
    assert _abi.profile_enable(0) == 0     # stage timing records events: off while a call is recorded
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _abi.check(lib.ckv_update_static(C.byref(b), C.c_void_p(torch.cuda.current_stream().cuda_stream)),
                   "ckv_update_static under capture")
    scratch = torch.zeros(1 << 14, device="cuda:0")
    for rep in range(8):                   # 8 x 24 tokens: the first ring of the 4 + 4 x 32-slot cache fills and evicts
        fresh_inputs()
        _abi.check(lib.ckv_update(C.byref(a), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "ckv_update")
        graph.replay()
        advance()
        scratch.add_(1.0).mul_(0.5)        # the program's own eager work between two replays
        same(f"replay {rep}")
    assert int(ref.start_indices[0].sum()) > 0 and int((~ref.mask[0]).sum()) > 32 * B * KVH
