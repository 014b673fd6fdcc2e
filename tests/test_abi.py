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
