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

from cascading_kv_cache_amd._abi import UpdateArgs, fill_update_args

from . import build as _build

_LIB = None


def _lib():
    global _LIB
    if _LIB is None:
        path = _build.OUT
        if not os.path.exists(path):
            path = _build.build()
        L = C.CDLL(path)
        L.ckv_oracle_update.argtypes = [C.POINTER(UpdateArgs)]
        L.ckv_oracle_update.restype = C.c_int
        _LIB = L
    return _LIB


def oracle_sink_cache(k, v, s, sink_k, sink_v, sink_mask, sink_pos, cache_k, cache_v, cache_s, mask, pos,
                      og_pos, do_cache, do_cache_every_n, stored_tokens, start_indices, stored_sinks,
                      num_sink, window_size, real_token_idx, max_seq_len, eager_fill):
    for t in (k, cache_k, stored_tokens):
        assert t.device.type == "cpu", "the oracle runs on host memory"
    a = fill_update_args(k, v, s, sink_k, sink_v, sink_mask, sink_pos, cache_k, cache_v, cache_s, mask, pos,
                         og_pos, do_cache_every_n, stored_tokens, start_indices, stored_sinks, num_sink,
                         window_size, real_token_idx, max_seq_len, eager_fill)
    rc = _lib().ckv_oracle_update(C.byref(a))
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
