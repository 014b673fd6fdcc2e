"""ctypes mirror of ``include/ckv.h`` and the loader of ``libckv.so``.

The structures here must stay field-for-field identical to the C header; the CPU test-suite
checks their sizes against ``ckv_sizeof_*`` helpers exported by the library.
"""
import ctypes as C
import os

import torch

I64 = C.c_int64
VP = C.c_void_p

CKV_F32, CKV_F16, CKV_BF16 = 0, 1, 2
CKV_REDUCE = {"mean": 0, "max": 1, "median": 2}

_DTYPES = {torch.float32: CKV_F32, torch.float16: CKV_F16, torch.bfloat16: CKV_BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"unsupported cache dtype {dtype}; expected float32, float16 or bfloat16")


class UpdateArgs(C.Structure):
    _fields_ = [
        ("k", VP), ("v", VP), ("kv_stride", I64 * 4),
        ("s", VP), ("s_stride", I64 * 3),
        ("sink_k", VP), ("sink_v", VP), ("sink_stride", I64 * 4),
        ("cache_k", VP), ("cache_v", VP), ("cache_stride", I64 * 4),
        ("cache_s", VP), ("cache_s_stride", I64 * 3),
        ("sink_mask", VP), ("sink_mask_stride", I64 * 3),
        ("mask", VP), ("mask_stride", I64 * 3),
        ("sink_pos", VP), ("sink_pos_stride", I64 * 3),
        ("pos", VP), ("pos_stride", I64 * 3),
        ("og_pos", VP), ("og_pos_stride", I64 * 3),
        ("stored_sinks", VP), ("stored_sinks_stride", I64 * 2),
        ("stored_tokens", VP), ("start_indices", VP), ("tracker_stride", I64 * 3),
        ("do_cache_every_n", VP), ("real_token_idx", VP),
        ("N", I64), ("H", I64), ("K", I64), ("HID", I64),
        ("num_sink", I64), ("window_size", I64), ("max_seq_len", I64),
        ("cascades", C.c_int32), ("eager_fill", C.c_int32), ("dtype", C.c_int32), ("reserved", C.c_int32),
        ("workspace", VP), ("workspace_bytes", I64),
    ]


class AttnArgs(C.Structure):
    _fields_ = [
        ("q", VP), ("q_stride", I64 * 4),
        ("k_new", VP), ("v_new", VP), ("kv_new_stride", I64 * 4),
        ("sink_k", VP), ("sink_v", VP), ("sink_stride", I64 * 4),
        ("cache_k", VP), ("cache_v", VP), ("cache_stride", I64 * 4),
        ("sink_mask", VP), ("mask", VP),
        ("q_pos", VP),
        ("sink_pos", VP), ("sink_pos_stride", I64 * 2),
        ("pos", VP), ("pos_stride", I64 * 2),
        ("pos_shift", I64),
        ("cache_s", VP), ("cache_s_stride", I64 * 3),
        ("out", VP), ("out_stride", I64 * 4),
        ("new_scores", VP), ("new_scores_stride", I64 * 3),
        ("lse", VP),
        ("B", I64), ("H", I64), ("KVH", I64), ("Q", I64), ("D", I64),
        ("num_sink", I64), ("S", I64),
        ("scale", C.c_float), ("rope_theta", C.c_float),
        ("inv_freq", VP),
        ("beta", C.c_double),
        ("head_reduction", C.c_int32), ("homogeneous_heads", C.c_int32),
        ("dtype", C.c_int32), ("filled_slots", C.c_int32),
        ("workspace", VP), ("workspace_bytes", I64),
    ]


class DenseArgs(C.Structure):
    _fields_ = [
        ("q", VP), ("q_stride", I64 * 4),
        ("k", VP), ("v", VP), ("kv_stride", I64 * 4),
        ("mask", VP),
        ("out", VP), ("out_stride", I64 * 4),
        ("scores", VP), ("scores_stride", I64 * 3),
        ("B", I64), ("H", I64), ("n_ctx", I64), ("n_kv", I64), ("D", I64),
        ("scale", C.c_float),
        ("beta", C.c_double),
        ("causal", C.c_int32), ("dtype", C.c_int32),
        ("workspace", VP), ("workspace_bytes", I64),
        ("lse", VP),
    ]


class DenseBwdArgs(C.Structure):
    _fields_ = [
        ("q", VP), ("q_stride", I64 * 4),
        ("k", VP), ("v", VP), ("kv_stride", I64 * 4),
        ("mask", VP),
        ("out", VP), ("out_stride", I64 * 4),
        ("lse", VP),
        ("dout", VP), ("dout_stride", I64 * 4),
        ("dq", VP), ("dq_stride", I64 * 4),
        ("dk", VP), ("dv", VP), ("dkv_stride", I64 * 4),
        ("B", I64), ("H", I64), ("n_ctx", I64), ("n_kv", I64), ("D", I64),
        ("scale", C.c_float), ("dtype", C.c_int32),
        ("workspace", VP), ("workspace_bytes", I64),
    ]


def set_strides(field, tensor_or_strides):
    strides = tensor_or_strides.stride() if hasattr(tensor_or_strides, "stride") else tensor_or_strides
    assert len(strides) == len(field), (len(strides), len(field))
    for i, s in enumerate(strides):
        field[i] = int(s)


def same_layout(a, b) -> bool:
    """Equal shapes and equal strides on every dimension that is actually stepped through
    (the stride of a size-1 dimension is arbitrary in torch)."""
    return a.shape == b.shape and all(sa == sb for n, sa, sb in zip(a.shape, a.stride(), b.stride()) if n > 1)


def fill_update_args(k, v, s, sink_k, sink_v, sink_mask, sink_pos, cache_k, cache_v, cache_s, mask, pos,
                     og_pos, do_cache_every_n, stored_tokens, start_indices, stored_sinks, num_sink,
                     window_size, real_token_idx, max_seq_len, eager_fill) -> UpdateArgs:
    """Describe the tensors of one ``sink_cache`` call (cascading_cache.py:962-985) for the C ABI.

    Applies the reference's own preconditions (cascading_cache.py:806-813); works for tensors
    on any device because only ``data_ptr``/``stride`` are read.
    """
    assert k.ndim == 4 and v.ndim == 4
    N, H, K, HID = k.shape
    assert v.shape == (N, H, K, HID)
    assert same_layout(k, v)
    assert same_layout(sink_k, sink_v)
    assert same_layout(cache_k, cache_v)
    assert same_layout(stored_tokens, start_indices)
    for t in (v, s, sink_k, sink_v, cache_k, cache_v, cache_s):
        if t.dtype != k.dtype:
            raise TypeError(f"all floating tensors must share one dtype, got {t.dtype} and {k.dtype}")
    for t in (sink_mask, mask):
        if t.dtype != torch.bool:
            raise TypeError("masks must be torch.bool")
    for t in (sink_pos, pos, og_pos, do_cache_every_n, stored_tokens, start_indices, stored_sinks, real_token_idx):
        if t.dtype != torch.int64:
            raise TypeError("index tensors must be torch.int64")
    if not do_cache_every_n.is_contiguous():
        raise ValueError("do_cache_every_n must be contiguous")
    # The kernel addresses every state tensor with the sizes of k: a chunk with more streams, heads or a
    # wider row than the cache holds would be written past the allocations.
    S, C_ = int(max_seq_len), int(stored_tokens.size(-1))
    want = {
        "cache_k": (cache_k, (H, S, HID)), "sink_k": (sink_k, (H, int(num_sink), HID)),
        "cache_s": (cache_s, (H, S)), "mask": (mask, (H, S)), "pos": (pos, (H, S)), "og_pos": (og_pos, (H, S)),
        "sink_mask": (sink_mask, (H, int(num_sink))), "sink_pos": (sink_pos, (H, int(num_sink))),
        "stored_tokens": (stored_tokens, (H, C_)), "stored_sinks": (stored_sinks, (H,)),
    }
    for name, (t, tail) in want.items():
        if tuple(t.shape[1:]) != tail or t.size(0) < N:
            raise ValueError(f"{name} has shape {tuple(t.shape)}; a chunk of shape {tuple(k.shape)} needs "
                             f"(>= {N}, {', '.join(str(x) for x in tail)})")
    if s.ndim != 3 or s.size(0) < N or s.size(1) < H or s.size(2) != K:
        raise ValueError(f"scores have shape {tuple(s.shape)}; expected ({N}, >= {H}, {K})")
    if do_cache_every_n.numel() != C_ or C_ * int(window_size) != S:
        raise ValueError("cascades * window_size must equal max_seq_len, one acceptance period per cascade")
    for t in (v, s, sink_k, cache_k, cache_s, mask, pos, og_pos, stored_tokens, stored_sinks, do_cache_every_n,
              real_token_idx):
        if t.device != k.device:
            raise ValueError(f"all tensors of an update must live on one device, got {t.device} and {k.device}")

    a = UpdateArgs()
    a.k, a.v, a.s = k.data_ptr(), v.data_ptr(), s.data_ptr()
    set_strides(a.kv_stride, k)
    set_strides(a.s_stride, s)
    a.sink_k, a.sink_v = sink_k.data_ptr(), sink_v.data_ptr()
    set_strides(a.sink_stride, sink_k)
    a.cache_k, a.cache_v = cache_k.data_ptr(), cache_v.data_ptr()
    set_strides(a.cache_stride, cache_k)
    a.cache_s = cache_s.data_ptr()
    set_strides(a.cache_s_stride, cache_s)
    a.sink_mask = sink_mask.data_ptr()
    set_strides(a.sink_mask_stride, sink_mask)
    a.mask = mask.data_ptr()
    set_strides(a.mask_stride, mask)
    a.sink_pos = sink_pos.data_ptr()
    set_strides(a.sink_pos_stride, sink_pos)
    a.pos = pos.data_ptr()
    set_strides(a.pos_stride, pos)
    a.og_pos = og_pos.data_ptr()
    set_strides(a.og_pos_stride, og_pos)
    a.stored_sinks = stored_sinks.data_ptr()
    set_strides(a.stored_sinks_stride, stored_sinks)
    a.stored_tokens, a.start_indices = stored_tokens.data_ptr(), start_indices.data_ptr()
    set_strides(a.tracker_stride, stored_tokens)
    a.do_cache_every_n = do_cache_every_n.data_ptr()
    a.real_token_idx = real_token_idx.data_ptr()
    a.N, a.H, a.K, a.HID = N, H, K, HID
    a.num_sink, a.window_size, a.max_seq_len = int(num_sink), int(window_size), int(max_seq_len)
    a.cascades = int(stored_tokens.size(-1))
    a.eager_fill = int(bool(eager_fill))
    a.dtype = dtype_code(k.dtype)
    a.workspace, a.workspace_bytes = None, 0
    return a


# ---------------------------------------------------------------------------------------------
# library loading
# ---------------------------------------------------------------------------------------------
_LIB = None
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libckv.so")


class CkvError(RuntimeError):
    pass


def lib():
    """Return the loaded ``libckv.so`` or raise: there is no CPU or eager fallback."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise CkvError(
                f"{LIB_PATH} is missing: build it with `python -m cascading_kv_cache_amd.build` "
                "(hipcc, --offload-arch=gfx950); there is no fallback path")
        L = C.CDLL(LIB_PATH)
        L.ckv_update.argtypes = [C.POINTER(UpdateArgs), VP]
        L.ckv_update.restype = C.c_int
        L.ckv_update_static.argtypes = [C.POINTER(UpdateArgs), VP]
        L.ckv_update_static.restype = C.c_int
        L.ckv_update_static_scratch_bytes.argtypes = []
        L.ckv_update_static_scratch_bytes.restype = I64
        L.ckv_update_workspace_bytes.argtypes = [I64, I64, I64, I64, C.c_int32]
        L.ckv_update_workspace_bytes.restype = I64
        L.ckv_attn.argtypes = [C.POINTER(AttnArgs), VP]
        L.ckv_attn.restype = C.c_int
        L.ckv_attn_workspace_bytes.argtypes = [I64, I64, I64, I64, I64, I64, I64, C.c_int32]
        L.ckv_attn_workspace_bytes.restype = I64
        L.ckv_attn_dense.argtypes = [C.POINTER(DenseArgs), VP]
        L.ckv_attn_dense.restype = C.c_int
        L.ckv_dense_workspace_bytes.argtypes = [I64, I64, I64, I64, I64, C.c_int32]
        L.ckv_dense_workspace_bytes.restype = I64
        L.ckv_attn_dense_bwd.argtypes = [C.POINTER(DenseBwdArgs), VP]
        L.ckv_attn_dense_bwd.restype = C.c_int
        L.ckv_dense_bwd_workspace_bytes.argtypes = [I64, I64, I64]
        L.ckv_dense_bwd_workspace_bytes.restype = I64
        L.ckv_chunk_positions.argtypes = [C.c_void_p, I64, I64, C.c_void_p, I64, I64, C.c_void_p, C.c_void_p]
        L.ckv_chunk_positions.restype = C.c_int
        L.ckv_profile_enable.argtypes = [C.c_int]
        L.ckv_profile_enable.restype = C.c_int
        L.ckv_profile_read.argtypes = [C.POINTER(C.c_double), C.POINTER(I64)]
        L.ckv_profile_read.restype = C.c_int
        L.ckv_strerror.argtypes = [C.c_int]
        L.ckv_strerror.restype = C.c_char_p
        L.ckv_abi_version.argtypes = []
        L.ckv_abi_version.restype = C.c_int
        _LIB = L
    return _LIB


STAGES = ("prep", "fwd", "scores", "finish", "decode", "decode_tail", "plan", "apply")


def profile_enable(on) -> int:
    """0 / False: off; 1 / True: every stage; 2: only the attention main kernels.  Returns the previous level."""
    return int(lib().ckv_profile_enable(int(on)))


def profile_read():
    """{stage: (milliseconds, launches)} accumulated since the last read (waits for the events)."""
    ms = (C.c_double * len(STAGES))()
    n = (I64 * len(STAGES))()
    check(lib().ckv_profile_read(ms, n), "ckv_profile_read")
    return {name: (ms[i], n[i]) for i, name in enumerate(STAGES)}


def check(status: int, what: str):
    if status != 0:
        raise CkvError(f"{what} failed: {lib().ckv_strerror(status).decode()} ({status})")
