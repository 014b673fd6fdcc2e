"""TEST INFRASTRUCTURE: Python face of the C update oracle plus a CPU cache-state container.

``oracle_sink_cache`` has the positional signature of the reference's ``sink_cache``
(cascade/models/cascading_cache.py:962-985) and runs ``ckv_oracle_update`` (the serial
per-token restatement in ``ckv_oracle_update.c``) on CPU tensors.

``OracleCache`` restates the state layout and bookkeeping of ``CascadingKVCache``
(cascade/models/cascading_cache.py:1187-1348): ``init_cache`` allocation, ``get_vals`` with its
sink shift, ``update`` and its counter ordering.
"""
import ctypes as C
import os

import torch

from . import build as _build

_LIB = None

ORACLE_DTYPE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


class OracleTensor(C.Structure):
    """``oracle_tensor`` of ckv_oracle_update.c: base pointer and element strides, outermost first."""
    _fields_ = [("ptr", C.c_void_p), ("stride", C.c_int64 * 4)]


_TENSOR_FIELDS = ("k", "v", "s", "sink_k", "sink_v", "sink_mask", "sink_pos", "cache_k", "cache_v", "cache_s",
                  "mask", "pos", "og_pos", "do_cache_every_n", "stored_tokens", "start_indices", "stored_sinks")
_SCALAR_FIELDS = ("num_sink", "window_size", "real_token_idx", "max_seq_len", "eager_fill", "n", "h", "k_len", "hid",
                  "cascades", "dtype")


class OracleUpdateDesc(C.Structure):
    """``oracle_update_desc`` of ckv_oracle_update.c: the arguments of ``sink_cache`` in the order of its
    signature (cascading_cache.py:962-985).  Deliberately not the library's argument struct: the oracle is
    described by code of its own, so a marshalling mistake on the product's side cannot cancel out."""
    _fields_ = [(name, OracleTensor) for name in _TENSOR_FIELDS] + [(name, C.c_int64) for name in _SCALAR_FIELDS]


def describe_update(k, v, s, sink_k, sink_v, sink_mask, sink_pos, cache_k, cache_v, cache_s, mask, pos, og_pos,
                    do_cache_every_n, stored_tokens, start_indices, stored_sinks, num_sink, window_size,
                    real_token_idx, max_seq_len, eager_fill) -> OracleUpdateDesc:
    """One record per tensor, taken from the tensor itself.  The reference kernel walks k and v, the two sink
    tensors, the two cache tensors and the two trackers with one set of strides each
    (cascading_cache.py:846-891), so pairs whose stepped strides differ are refused here."""
    tensors = dict(k=k, v=v, s=s, sink_k=sink_k, sink_v=sink_v, sink_mask=sink_mask, sink_pos=sink_pos,
                   cache_k=cache_k, cache_v=cache_v, cache_s=cache_s, mask=mask, pos=pos, og_pos=og_pos,
                   do_cache_every_n=do_cache_every_n, stored_tokens=stored_tokens, start_indices=start_indices,
                   stored_sinks=stored_sinks)
    for a, b in (("k", "v"), ("sink_k", "sink_v"), ("cache_k", "cache_v"), ("stored_tokens", "start_indices")):
        ta, tb = tensors[a], tensors[b]
        assert ta.shape == tb.shape, (a, b)
        for size, sa, sb in zip(ta.shape, ta.stride(), tb.stride()):
            assert size <= 1 or sa == sb, f"{a} and {b} must share strides"
    floating = ("k", "v", "s", "sink_k", "sink_v", "cache_k", "cache_v", "cache_s")
    assert all(tensors[n].dtype == k.dtype for n in floating)
    assert sink_mask.dtype == torch.bool and mask.dtype == torch.bool
    integer = ("sink_pos", "pos", "og_pos", "do_cache_every_n", "stored_tokens", "start_indices", "stored_sinks")
    assert all(tensors[n].dtype == torch.int64 for n in integer)
    d = OracleUpdateDesc()
    for name, t in tensors.items():
        assert t.device.type == "cpu", "the oracle runs on host memory"
        rec = getattr(d, name)
        rec.ptr = t.data_ptr()
        for i, st in enumerate(t.stride()):
            rec.stride[i] = st
    d.num_sink, d.window_size, d.max_seq_len = int(num_sink), int(window_size), int(max_seq_len)
    d.real_token_idx = int(real_token_idx)
    d.eager_fill = 1 if eager_fill else 0
    d.n, d.h, d.k_len, d.hid = k.shape
    d.cascades = stored_tokens.shape[-1]
    d.dtype = ORACLE_DTYPE[k.dtype]
    return d


def _lib():
    global _LIB
    if _LIB is None:
        path = _build.OUT
        if not os.path.exists(path):
            path = _build.build()
        L = C.CDLL(path)
        L.ckv_oracle_update.argtypes = [C.POINTER(OracleUpdateDesc)]
        L.ckv_oracle_update.restype = C.c_int
        L.ckv_oracle_sizeof_desc.argtypes = []
        L.ckv_oracle_sizeof_desc.restype = C.c_int64
        assert L.ckv_oracle_sizeof_desc() == C.sizeof(OracleUpdateDesc)
        _LIB = L
    return _LIB


def oracle_sink_cache(k, v, s, sink_k, sink_v, sink_mask, sink_pos, cache_k, cache_v, cache_s, mask, pos,
                      og_pos, do_cache, do_cache_every_n, stored_tokens, start_indices, stored_sinks,
                      num_sink, window_size, real_token_idx, max_seq_len, eager_fill):
    d = describe_update(k, v, s, sink_k, sink_v, sink_mask, sink_pos, cache_k, cache_v, cache_s, mask, pos,
                        og_pos, do_cache_every_n, stored_tokens, start_indices, stored_sinks, num_sink,
                        window_size, real_token_idx, max_seq_len, eager_fill)
    rc = _lib().ckv_oracle_update(C.byref(d))
    if rc != 0:
        raise RuntimeError(f"ckv_oracle_update returned {rc}")
    return k, v


CASCADE_FUNCS = ("pow2", "pow2-1", "pow2-1-4", "pow2-2-4", "pow2-3-4", "1-then-2", "pow3", "pow4", "iplus1")


def acceptance_periods(cascade_func: str, c: int):
    """do_cache_every_n of one layer (cascading_cache.py:1201-1244)."""
    if cascade_func == "pow2":
        return [2**i for i in range(c)]
    if cascade_func == "pow2-1":
        return [1] * (c - 1) + [2**i for i in range(c - 1, c)]
    if cascade_func in ("pow2-1-4", "pow2-2-4", "pow2-3-4"):
        ones = {"pow2-1-4": 3, "pow2-2-4": 2, "pow2-3-4": 1}[cascade_func] * (c // 4)
        return [1] * ones + [2**i for i in range(ones, c)]
    if cascade_func == "1-then-2":
        return [1] + [2] * (c - 1)
    if cascade_func == "pow3":
        return [3**i for i in range(c)]
    if cascade_func == "pow4":
        return [4**i for i in range(c)]
    if cascade_func == "iplus1":
        return [i + 1 for i in range(c)]
    raise ValueError(f"unknown cascade func: {cascade_func}")


class OracleCache:
    """Single-layer CPU state with the tensors of cascading_cache.py:1196-1276."""

    def __init__(self, window_length, num_sink_tokens, max_batch_size, heads, dim, max_seq_len,
                 dtype=torch.float32, cascade_func="pow2", eager_fill=True, beta=0.9999999):
        if max_seq_len % window_length != 0:
            raise ValueError("window length must evenly divide max seq len")
        B, H, D, S, NS = max_batch_size, heads, dim, max_seq_len, num_sink_tokens
        self.window_length, self.num_sink_tokens, self.max_seq_len = window_length, NS, S
        self.cascades = S // window_length
        self.dtype, self.eager_fill, self.beta = dtype, eager_fill, beta
        self.max_batch_size, self.heads, self.dim = B, H, D
        self.seen_tokens = torch.zeros((), dtype=torch.long)
        self.do_cache = torch.ones(self.cascades, dtype=torch.bool)
        self.do_cache_every_n = torch.tensor(acceptance_periods(cascade_func, self.cascades), dtype=torch.long)
        self.stored_tokens = torch.zeros(B, H, self.cascades, dtype=torch.long)
        self.start_indices = torch.zeros(B, H, self.cascades, dtype=torch.long)
        self.stored_sinks = torch.zeros(B, H, dtype=torch.long)
        self.pos = torch.zeros(B, H, S, dtype=torch.long)
        self.og_pos = torch.zeros(B, H, S, dtype=torch.long)
        self.sink_pos = torch.zeros(B, H, NS, dtype=torch.long)
        self.key_cache = torch.zeros(B, H, S, D, dtype=dtype)
        self.value_cache = torch.zeros(B, H, S, D, dtype=dtype)
        self.score_cache = torch.zeros(B, H, S, dtype=dtype)
        self.sink_keys = torch.zeros(B, H, NS, D, dtype=dtype)
        self.sink_values = torch.zeros(B, H, NS, D, dtype=dtype)
        self.mask = torch.ones(B, H, S, dtype=torch.bool)
        self.sink_mask = torch.ones(B, H, NS, dtype=torch.bool)

    def get_vals(self):
        """cascading_cache.py:1278-1295."""
        shift = self.num_sink_tokens if int(self.seen_tokens) > self.num_sink_tokens else 0
        return (self.sink_keys, self.sink_values, self.sink_pos[:1, 0], self.sink_mask, self.key_cache,
                self.value_cache, self.pos[:1, 0] + shift, self.mask, self.og_pos)

    def update(self, key_states, value_states, score_states=None):
        """cascading_cache.py:1297-1348: zero scores by default, counter bumped after the kernel."""
        if score_states is None:
            score_states = torch.zeros(self.max_batch_size, self.heads, key_states.size(2), dtype=key_states.dtype)
        oracle_sink_cache(key_states, value_states, score_states, self.sink_keys, self.sink_values,
                          self.sink_mask, self.sink_pos, self.key_cache, self.value_cache, self.score_cache,
                          self.mask, self.pos, self.og_pos, self.do_cache, self.do_cache_every_n,
                          self.stored_tokens, self.start_indices, self.stored_sinks, self.num_sink_tokens,
                          self.window_length, self.seen_tokens, self.max_seq_len, self.eager_fill)
        self.seen_tokens += key_states.shape[-2]
        return self.get_vals()

    def state_dict(self):
        names = ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask",
                 "pos", "og_pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")
        return {n: getattr(self, n) for n in names}
