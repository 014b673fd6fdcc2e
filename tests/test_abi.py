"""CPU checks of the C-ABI boundary: libckv.so loads, exports every entry point that include/ckv.h
declares, the ctypes mirrors match the C structs, and argument validation answers with status
codes before anything touches a GPU."""
import ctypes as C
import os
import re

import pytest
import torch

from cascading_kv_cache_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_abi.LIB_PATH):
        from cascading_kv_cache_amd import build

        build.build(verbose=False)
    return _abi.lib()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ckv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ckv_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("ckv_update", "ckv_update_workspace_bytes", "ckv_attn", "ckv_attn_workspace_bytes", "ckv_attn_dense",
                 "ckv_dense_workspace_bytes", "ckv_strerror", "ckv_abi_version", "ckv_profile_enable",
                 "ckv_profile_read", "ckv_chunk_positions", "ckv_update_static", "ckv_attn_dense_bwd",
                 "ckv_dense_bwd_workspace_bytes"):
        assert must in names


def test_library_exports_every_declared_symbol(lib):
    raw = C.CDLL(_abi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(raw, name), f"{name} is declared in include/ckv.h but not exported"
    assert lib.ckv_abi_version() == 2


def test_ctypes_mirrors_match_struct_sizes(lib):
    raw = C.CDLL(_abi.LIB_PATH)
    for fn, struct in (("ckv_sizeof_update_args", _abi.UpdateArgs), ("ckv_sizeof_attn_args", _abi.AttnArgs),
                       ("ckv_sizeof_dense_args", _abi.DenseArgs), ("ckv_sizeof_dense_bwd_args", _abi.DenseBwdArgs)):
        f = getattr(raw, fn)
        f.restype = C.c_int64
        assert f() == C.sizeof(struct), fn


def test_status_strings(lib):
    seen = set()
    for code in range(0, -9, -1):
        text = lib.ckv_strerror(code).decode()
        assert text and text not in seen
        seen.add(text)
    assert "unknown" in lib.ckv_strerror(-99).decode()


def test_workspace_sizes(lib):
    assert lib.ckv_update_workspace_bytes(2, 8, 2048, 16384, 8) >= 2 * 8 * (2048 + 16384) * 4
    assert lib.ckv_update_workspace_bytes(0, 8, 1, 16, 1) == 0
    small = lib.ckv_attn_workspace_bytes(1, 8, 2, 16, 128, 4, 64, _abi.CKV_BF16)
    big = lib.ckv_attn_workspace_bytes(2, 32, 8, 2048, 128, 64, 16384, _abi.CKV_BF16)
    assert 0 < small < big
    assert lib.ckv_attn_workspace_bytes(1, 8, 2, 1, 128, 4, 64, _abi.CKV_BF16) > 0  # decode
    assert lib.ckv_dense_workspace_bytes(1, 2, 128, 256, 64, _abi.CKV_F16) > 0
    assert lib.ckv_dense_workspace_bytes(1, 2, 128, 64, 64, _abi.CKV_F16) == 0  # n_kv < n_ctx


def test_update_argument_validation_needs_no_gpu(lib):
    assert lib.ckv_update(None, None) == -1  # CKV_ERR_NULL
    a = _abi.UpdateArgs()
    a.dtype = 7
    assert lib.ckv_update(C.byref(a), None) == -4  # CKV_ERR_DTYPE
    a.dtype = _abi.CKV_BF16
    a.N, a.H, a.K, a.HID = 1, 1, 1, 128
    a.window_size, a.cascades, a.max_seq_len = 4, 2, 9  # 2 * 4 != 9
    assert lib.ckv_update(C.byref(a), None) == -2  # CKV_ERR_SHAPE
    a.max_seq_len = 8
    assert lib.ckv_update(C.byref(a), None) == -1  # state pointers missing
    a.cascades, a.max_seq_len = 65, 260
    assert lib.ckv_update(C.byref(a), None) == -2  # more cascades than the planner supports


def test_attention_argument_validation_needs_no_gpu(lib):
    assert lib.ckv_attn(None, None) == -1
    a = _abi.AttnArgs()
    a.dtype = _abi.CKV_BF16
    a.B, a.H, a.KVH, a.Q, a.D = 1, 6, 4, 8, 128  # 6 % 4 != 0
    assert lib.ckv_attn(C.byref(a), None) == -2
    a.H = 8
    a.head_reduction = 5
    assert lib.ckv_attn(C.byref(a), None) == -2
    a.head_reduction = 0
    assert lib.ckv_attn(C.byref(a), None) == -1  # q / k_new / ... missing
    assert lib.ckv_attn_dense(None, None) == -1
    assert lib.ckv_chunk_positions(None, 0, 0, None, 0, 4, None, None) == -1   # no output
    assert lib.ckv_chunk_positions(None, 0, 0, None, 0, 0, 8, None) == -2      # empty chunk (checked before any launch)
    d = _abi.DenseArgs()
    d.dtype = _abi.CKV_F16
    d.B, d.H, d.n_ctx, d.n_kv, d.D = 1, 1, 16, 8, 64
    assert lib.ckv_attn_dense(C.byref(d), None) == -2
    assert lib.ckv_attn_dense_bwd(None, None) == -1
    g = _abi.DenseBwdArgs()
    g.dtype = _abi.CKV_F16
    g.B, g.H, g.n_ctx, g.n_kv, g.D = 1, 1, 16, 8, 64
    assert lib.ckv_attn_dense_bwd(C.byref(g), None) == -2    # fewer keys than queries
    g.n_kv, g.D = 32, 256
    assert lib.ckv_attn_dense_bwd(C.byref(g), None) == -6    # head size beyond what the backward kernels tile
    g.D = 64
    assert lib.ckv_attn_dense_bwd(C.byref(g), None) == -1    # tensors missing
    assert lib.ckv_dense_bwd_workspace_bytes(2, 4, 100) >= 2 * 4 * 100 * 4


def test_fill_update_args_enforces_reference_preconditions():
    k = torch.zeros(1, 2, 3, 8)
    st = dict(sink_k=torch.zeros(1, 2, 2, 8), sink_v=torch.zeros(1, 2, 2, 8), sink_mask=torch.ones(1, 2, 2, dtype=torch.bool),
              sink_pos=torch.zeros(1, 2, 2, dtype=torch.long), cache_k=torch.zeros(1, 2, 4, 8),
              cache_v=torch.zeros(1, 2, 4, 8), cache_s=torch.zeros(1, 2, 4), mask=torch.ones(1, 2, 4, dtype=torch.bool),
              pos=torch.zeros(1, 2, 4, dtype=torch.long), og_pos=torch.zeros(1, 2, 4, dtype=torch.long),
              do_cache_every_n=torch.tensor([1, 2]), stored_tokens=torch.zeros(1, 2, 2, dtype=torch.long),
              start_indices=torch.zeros(1, 2, 2, dtype=torch.long), stored_sinks=torch.zeros(1, 2, dtype=torch.long))

    def fill(**over):
        d = dict(st)
        d.update(over)
        return _abi.fill_update_args(k, over.get("v", k.clone()), over.get("s", torch.zeros(1, 2, 3)), d["sink_k"],
                                     d["sink_v"], d["sink_mask"], d["sink_pos"], d["cache_k"], d["cache_v"],
                                     d["cache_s"], d["mask"], d["pos"], d["og_pos"], d["do_cache_every_n"],
                                     d["stored_tokens"], d["start_indices"], d["stored_sinks"], 2, 2,
                                     torch.zeros((), dtype=torch.long), 4, True)

    a = fill()
    assert (a.N, a.H, a.K, a.HID, a.cascades, a.dtype) == (1, 2, 3, 8, 2, _abi.CKV_F32)
    with pytest.raises(AssertionError):  # k and v must share strides (cascading_cache.py:810)
        fill(v=torch.zeros(1, 3, 2, 8).transpose(1, 2))
    with pytest.raises(TypeError):
        fill(s=torch.zeros(1, 2, 3, dtype=torch.float16))
    with pytest.raises(TypeError):
        fill(mask=torch.ones(1, 2, 4))
    with pytest.raises(TypeError):
        fill(pos=torch.zeros(1, 2, 4, dtype=torch.int32))


def test_memoised_update_arguments_follow_reassigned_state_tensors():
    """The reference reassigns ``score_cache[l]`` every call (cascade_attention.py:222-224).  The memoised
    argument block holds raw pointers, so it must follow the tensor the cache holds NOW, also when a freed
    tensor's Python id is handed to a new one."""
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    c = CascadingKVCache(window_length=4, num_sink_tokens=2, max_batch_size=1, heads=2, dim=8, max_seq_len=8,
                         device="cpu", dtype=torch.float32, layers=1, verbose=False)
    k, v, s = torch.zeros(1, 2, 3, 8), torch.zeros(1, 2, 3, 8), torch.zeros(1, 2, 3)
    keep = []  # keeps every tensor alive so each reassignment lands at a new address
    for step in range(80):  # more steps than the memo holds entries
        fresh = c.score_cache[0] * 0.5 + 1.0
        keep.append(fresh)
        c.score_cache[0] = fresh
        a = c._update_args(k, v, s, 0)
        assert a.cache_s == fresh.data_ptr(), f"step {step}: stale score-cache pointer in the argument block"
        assert a.cache_k == c.key_cache[0].data_ptr() and a.k == k.data_ptr()
    # the same address again -> the same block is reused, with the input pointers refreshed
    k2 = torch.ones(1, 2, 3, 8)
    b = c._update_args(k2, v, s, 0)
    assert b is a and b.k == k2.data_ptr()
    # ids may repeat, addresses of live tensors cannot: drop and re-create without keeping
    for step in range(80):
        c.score_cache[0] = c.score_cache[0] * 0.5
        assert c._update_args(k, v, s, 0).cache_s == c.score_cache[0].data_ptr()


def test_chunk_is_checked_against_the_cache_before_any_pointer_leaves():
    from cascading_kv_cache_amd.cascade_attention import check_against_cache
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    c = CascadingKVCache(window_length=4, num_sink_tokens=2, max_batch_size=2, heads=2, dim=8, max_seq_len=8,
                         device="cpu", dtype=torch.float16, layers=1, verbose=False)

    def chunk(B=2, H=4, KVH=2, Q=3, D=8, dtype=torch.float16):
        return torch.zeros(B, H, Q, D, dtype=dtype), torch.zeros(B, KVH, Q, D, dtype=dtype), torch.zeros(B, KVH, Q, D, dtype=dtype)

    check_against_cache(*chunk(), c, 0)
    check_against_cache(*chunk(B=1), c, 0)                    # fewer streams than the cache holds is fine
    for bad in (dict(B=3), dict(KVH=1, H=4), dict(D=16), dict(H=3)):
        with pytest.raises(ValueError):
            check_against_cache(*chunk(**bad), c, 0)
    with pytest.raises(TypeError):                            # a bf16 chunk over an fp16 cache is not reinterpreted
        check_against_cache(*chunk(dtype=torch.bfloat16), c, 0)
    with pytest.raises(ValueError):
        check_against_cache(*chunk(), c, 1)
    # the update operator checks the same sizes
    k = torch.zeros(3, 2, 3, 8, dtype=torch.float16)
    with pytest.raises(ValueError):
        c._update_args(k, k.clone(), torch.zeros(3, 2, 3, dtype=torch.float16), 0)
    k = torch.zeros(2, 2, 3, 16, dtype=torch.float16)
    with pytest.raises(ValueError):
        c._update_args(k, k.clone(), torch.zeros(2, 2, 3, dtype=torch.float16), 0)
    k = torch.zeros(2, 2, 3, 8, dtype=torch.float16)
    with pytest.raises(ValueError):
        c._update_args(k, k.clone(), torch.zeros(2, 1, 3, dtype=torch.float16), 0)


# ---------------------------------------------------------------------------------------------
# The oracle describes its arguments with code of its own (oracle/update.py:describe_update), the
# library with _abi.fill_update_args.  Both are fed deliberately odd layouts and must agree field
# by field; the oracle must also give the same result on those layouts as on contiguous copies.
# ---------------------------------------------------------------------------------------------
def _odd_layout_state(seed=0, N=2, KVH=3, H=6, K=5, D=4, NS=3, W=4, Cc=2, dtype=torch.float32):
    """Every tensor of one sink_cache call as a non-contiguous view: scores with H > KVH heads in a
    transposed layout (the caller of cascade_attention.py:331-339 repeats and hands over (B, H, q)),
    caches and trackers cut out of larger buffers, incoming rows with a padded last dimension."""
    g = torch.Generator().manual_seed(seed)
    S = W * Cc

    def cut(*shape, dt=dtype, pad=2):
        big = torch.zeros(*(s + pad for s in shape), dtype=dt)
        return big[tuple(slice(1, 1 + s) for s in shape)]

    t = {}
    t["k"] = torch.randn(N, K, KVH, D + 3, generator=g).to(dtype).permute(0, 2, 1, 3)[..., 1:1 + D]
    t["v"] = torch.randn(N, K, KVH, D + 3, generator=g).to(dtype).permute(0, 2, 1, 3)[..., 1:1 + D]
    t["s"] = torch.rand(K, N, H, generator=g).to(dtype).permute(1, 2, 0)       # (N, H, K), K outermost in memory
    t["sink_k"], t["sink_v"] = cut(N, KVH, NS, D), cut(N, KVH, NS, D)
    t["cache_k"], t["cache_v"] = cut(N, KVH, S, D), cut(N, KVH, S, D)
    t["cache_s"] = cut(N, KVH, S)
    t["sink_mask"], t["mask"] = cut(N, KVH, NS, dt=torch.bool), cut(N, KVH, S, dt=torch.bool)
    t["sink_mask"].fill_(True)
    t["mask"].fill_(True)
    t["sink_pos"], t["pos"], t["og_pos"] = (cut(N, KVH, NS, dt=torch.long), cut(N, KVH, S, dt=torch.long),
                                            cut(N, KVH, S, dt=torch.long))
    t["stored_tokens"], t["start_indices"] = cut(N, KVH, Cc, dt=torch.long), cut(N, KVH, Cc, dt=torch.long)
    t["stored_sinks"] = cut(N, KVH, dt=torch.long)
    t["do_cache_every_n"] = torch.tensor([1, 2][:Cc], dtype=torch.long)
    return t, dict(num_sink=NS, window_size=W, max_seq_len=S)


_ORDER = ("k", "v", "s", "sink_k", "sink_v", "sink_mask", "sink_pos", "cache_k", "cache_v", "cache_s", "mask", "pos",
          "og_pos", "do_cache_every_n", "stored_tokens", "start_indices", "stored_sinks")


def test_oracle_and_library_describe_odd_layouts_alike():
    from oracle.update import describe_update

    t, sc = _odd_layout_state()
    seen = torch.tensor(0, dtype=torch.long)
    args = [t[n] for n in _ORDER]
    lib_a = _abi.fill_update_args(*args, sc["num_sink"], sc["window_size"], seen, sc["max_seq_len"], True)
    ora = describe_update(*args, sc["num_sink"], sc["window_size"], seen, sc["max_seq_len"], True)
    # which field of the library's struct carries the pointer / the strides of which tensor
    pairs = {"k": ("k", "kv_stride"), "v": ("v", "kv_stride"), "s": ("s", "s_stride"),
             "sink_k": ("sink_k", "sink_stride"), "sink_v": ("sink_v", "sink_stride"),
             "cache_k": ("cache_k", "cache_stride"), "cache_v": ("cache_v", "cache_stride"),
             "cache_s": ("cache_s", "cache_s_stride"), "sink_mask": ("sink_mask", "sink_mask_stride"),
             "mask": ("mask", "mask_stride"), "sink_pos": ("sink_pos", "sink_pos_stride"), "pos": ("pos", "pos_stride"),
             "og_pos": ("og_pos", "og_pos_stride"), "stored_sinks": ("stored_sinks", "stored_sinks_stride"),
             "stored_tokens": ("stored_tokens", "tracker_stride"), "start_indices": ("start_indices", "tracker_stride"),
             "do_cache_every_n": ("do_cache_every_n", None)}
    for name, (ptr_field, stride_field) in pairs.items():
        rec = getattr(ora, name)
        assert getattr(lib_a, ptr_field) == rec.ptr == t[name].data_ptr(), name
        if stride_field is None:
            continue
        got = list(getattr(lib_a, stride_field))
        for dim, size in enumerate(t[name].shape):
            if size > 1:  # the stride of a size-1 dimension is arbitrary
                assert got[dim] == rec.stride[dim] == t[name].stride(dim), (name, dim)
    assert (lib_a.N, lib_a.H, lib_a.K, lib_a.HID) == (ora.n, ora.h, ora.k_len, ora.hid) == tuple(t["k"].shape)
    assert (lib_a.num_sink, lib_a.window_size, lib_a.max_seq_len, lib_a.cascades) == (
        ora.num_sink, ora.window_size, ora.max_seq_len, ora.cascades)
    assert lib_a.eager_fill == ora.eager_fill == 1
    assert lib_a.dtype == _abi.CKV_F32 and ora.dtype == 0
    # the scores really are laid out with the token index outermost, and with more heads than the cache has
    assert t["s"].stride() == (6, 1, 12) and t["s"].size(1) > t["k"].size(1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_oracle_result_does_not_depend_on_the_layout(dtype):
    """Three calls on the odd layouts against the same calls on contiguous copies."""
    from oracle.update import oracle_sink_cache

    t, sc = _odd_layout_state(seed=3, dtype=dtype)
    flat = {n: x.clone().contiguous() for n, x in t.items()}
    seen = 0
    g = torch.Generator().manual_seed(9)
    for call in range(3):
        for n in ("k", "v", "s"):
            fresh = torch.rand(t[n].shape, generator=g).to(dtype)
            t[n].copy_(fresh)
            flat[n].copy_(fresh)
        for side in (t, flat):
            oracle_sink_cache(*[side[n] for n in _ORDER[:13]], None, *[side[n] for n in _ORDER[13:]],
                              sc["num_sink"], sc["window_size"], torch.tensor(seen), sc["max_seq_len"], True)
        seen += t["k"].size(2)
        for n in _ORDER[3:]:
            assert torch.equal(t[n], flat[n]), (call, n)
    assert not t["mask"].all() and t["stored_sinks"].eq(sc["num_sink"]).all()
