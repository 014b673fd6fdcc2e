"""Host-side mirror of the reference's cache operator and cache object.

``sink_cache`` keeps the positional signature of the reference operator
(cascade/models/cascading_cache.py:962-987) and forwards to ``ckv_update`` in ``libckv.so``;
``CascadingKVCache`` keeps the constructor, attributes and methods of the reference class
(cascade/models/cascading_cache.py:1031-1348) without depending on ``transformers``.
There is no CPU path: tensors must live on a HIP device and the library must be built.
"""
import ctypes as C
from typing import List, Optional, Union

import torch
from torch import Tensor

from . import _abi

_WORKSPACES = {}


_COUNTER_TABLES = {}
COUNTER_TABLE_ENTRIES = 1 << 21


def _counter_table(device) -> Tensor:
    """``0, 1, 2, ...`` as int64 on ``device`` (16 MiB, built once): element n is a device-resident n."""
    device = torch.device(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    t = _COUNTER_TABLES.get(key)
    if t is None:
        t = torch.arange(COUNTER_TABLE_ENTRIES, dtype=torch.long, device=device)
        _COUNTER_TABLES[key] = t
    return t


def workspace(device: torch.device, nbytes: int, stream: int = 0) -> Tensor:
    """Scratch for one library call: one buffer per (device, stream), grown on demand.  Calls on one
    stream run in order, so they can share a buffer; calls on different streams of a device may
    overlap and get buffers of their own.  ``stream`` is the raw stream handle (0: the null stream).
    A buffer that is outgrown is dropped only after the stream has passed the calls that used it
    (torch's caching allocator keeps a freed block tied to the stream it was allocated on)."""
    key = (device.type, device.index, int(stream))
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = buf
    return buf


def _require_device(t: Tensor, what: str):
    if t.device.type != "cuda":
        raise _abi.CkvError(f"{what} lives on {t.device}: libckv only runs on a HIP device (no CPU fallback)")


def sink_cache(
    k: Tensor, v: Tensor, s: Tensor,
    sink_k: Tensor, sink_v: Tensor, sink_mask: Tensor, sink_pos: Tensor,
    cache_k: Tensor, cache_v: Tensor, cache_s: Tensor,
    mask: Tensor, pos: Tensor, og_pos: Tensor,
    do_cache: Tensor, do_cache_every_n: Tensor,
    stored_tokens: Tensor, start_indices: Tensor, stored_sinks: Tensor,
    num_sink, window_size, real_token_idx, max_seq_len, eager_fill,
    BENCHMARK: bool = False,
):
    """Drop-in for ``sink_cache`` (cascading_cache.py:962-1028): mutates the 13 state tensors in
    place and returns ``(k, v)``.  ``do_cache`` is accepted and ignored, as in the reference
    kernel (cascading_cache.py:204, 281, 361)."""
    _require_device(k, "k")
    lib = _abi.lib()
    if BENCHMARK:
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
    a = _abi.fill_update_args(k, v, s, sink_k, sink_v, sink_mask, sink_pos, cache_k, cache_v, cache_s, mask, pos,
                              og_pos, do_cache_every_n, stored_tokens, start_indices, stored_sinks, num_sink,
                              window_size, real_token_idx, max_seq_len, eager_fill)
    need = lib.ckv_update_workspace_bytes(a.N, a.H, a.K, a.max_seq_len, a.cascades)
    with torch.cuda.device(k.device):
        stream = torch.cuda.current_stream(k.device).cuda_stream
        ws = workspace(k.device, need, stream)
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
        _abi.check(lib.ckv_update(C.byref(a), C.c_void_p(stream)), "ckv_update")
    if BENCHMARK:
        ev1.record()
        torch.cuda.synchronize()
        print(ev0.elapsed_time(ev1))
    return k, v


def acceptance_periods(cascade_func: str, cascades: int) -> List[int]:
    """The nine named acceptance schedules of cascading_cache.py:1201-1244."""
    c = cascades
    if cascade_func == "pow2":
        return [2 ** i for i in range(c)]
    if cascade_func == "pow2-1":
        return [1] * (c - 1) + [2 ** (c - 1)] if c > 0 else []
    if cascade_func in ("pow2-1-4", "pow2-2-4", "pow2-3-4"):
        ones = {"pow2-1-4": 3, "pow2-2-4": 2, "pow2-3-4": 1}[cascade_func] * (c // 4)
        return [1] * ones + [2 ** i for i in range(ones, c)]
    if cascade_func == "1-then-2":
        return [1] + [2] * (c - 1)
    if cascade_func == "pow3":
        return [3 ** i for i in range(c)]
    if cascade_func == "pow4":
        return [4 ** i for i in range(c)]
    if cascade_func == "iplus1":
        return [i + 1 for i in range(c)]
    raise ValueError(f"unknown cascade func: {cascade_func}")


class CascadingKVCache:
    """Per-layer sink + cascade state with the interface of the reference class
    (cascading_cache.py:1031-1348).  Tensors have the reference's shapes and dtypes
    (cascading_cache.py:1196-1276) so code that reads them keeps working."""

    def __init__(
        self,
        window_length: Union[int, List[int]] = 8,
        num_sink_tokens: int = 4,
        max_batch_size: int = 1,
        heads: int = 16,
        dim: int = 128,
        max_seq_len: Union[int, List[int]] = 32,
        device: torch.device = "cpu",
        dtype: torch.dtype = torch.float16,
        cascade_func: str = "pow2",
        head_reduction: str = "mean",
        layers: int = 32,
        eager_fill: bool = True,
        verbose: bool = True,
    ) -> None:
        # one size for every layer, or one per layer: both arguments in the same form (cascading_cache.py:1050-1057)
        per_layer = [isinstance(x, (list, tuple)) for x in (window_length, max_seq_len)]
        if per_layer[0] != per_layer[1]:
            raise ValueError("window_length and max_seq_len must both be integers or both be per-layer lists, got "
                             f"{type(window_length).__name__} and {type(max_seq_len).__name__}")
        if per_layer[0]:
            windows, lengths = [int(w) for w in window_length], [int(s) for s in max_seq_len]
            if len(windows) != layers or len(lengths) != layers:
                raise ValueError(f"per-layer sizes need {layers} entries, got {len(windows)} and {len(lengths)}")
        else:
            windows, lengths = [int(window_length)] * layers, [int(max_seq_len)] * layers
        bad = [l for l in range(layers) if windows[l] <= 0 or lengths[l] % windows[l] != 0]
        if bad:
            raise ValueError(f"max_seq_len must be a whole number of windows in every layer; layers {bad} have "
                             f"windows {[windows[l] for l in bad]} and lengths {[lengths[l] for l in bad]}")

        self.window_length, self.max_seq_len = windows, lengths
        self.cascades = [s // w for s, w in zip(lengths, windows)]
        self.num_sink_tokens = num_sink_tokens
        self.max_batch_size, self.heads, self.dim, self.layers = max_batch_size, heads, dim, layers
        self.bh = max_batch_size * heads
        self.device, self.dtype = device, dtype
        self.cascade_func, self.head_reduction, self.eager_fill = cascade_func, head_reduction, eager_fill
        self.verbose = verbose
        self._seen_tokens = 0
        self.init_cache(self.device)

    def __repr__(self):
        return (f"CascadingKVCache(layers={self.layers}, batch={self.max_batch_size}, heads={self.heads}, "
                f"dim={self.dim}, sinks={self.num_sink_tokens}, cascades={self.cascades}, slots={self.max_seq_len})")

    def __getitem__(self, layer_idx: int):
        return self.get_vals(layer_idx)

    def __iter__(self):
        for layer_idx in range(len(self)):
            yield self.get_vals(layer_idx)

    def __len__(self):
        return self.layers

    # the HF cache methods the reference leaves unimplemented (cascading_cache.py:1126-1162)
    def to_legacy_cache(self):
        raise NotImplementedError()

    @classmethod
    def from_legacy_cache(cls, past_key_values=None):
        raise NotImplementedError()

    def crop(self, max_length: int):
        raise NotImplementedError()

    def batch_split(self, full_batch_size: int, split_size: int):
        raise NotImplementedError()

    @classmethod
    def from_batch_splits(cls, splits):
        raise NotImplementedError()

    def batch_repeat_interleave(self, repeats: int):
        raise NotImplementedError()

    def batch_select_indices(self, indices: torch.Tensor):
        raise NotImplementedError()

    def reorder_cache(self, beam_idx: torch.LongTensor):
        raise NotImplementedError()

    @property
    def seen_tokens(self):
        raise NotImplementedError()

    def get_seq_length(self, layer_idx: Optional[int] = 0, cascade_idx: Optional[int] = -1) -> int:
        stored_sinks = self.stored_sinks[layer_idx][0, 0].item()
        stored_tokens = self.stored_tokens[layer_idx][0, 0].sum().item()
        return stored_sinks + stored_tokens

    def get_max_length(self) -> Optional[int]:
        return self.max_seq_len[0]

    def reset(self, verbose=True):
        if verbose:
            print(f"RESET HIP CACHE {self.cascade_func=}")
        self._seen_tokens = 0
        self._generation += 1   # a step recorded into a graph before the reset no longer describes this cache
        self._seen_host = [0 for _ in range(self.layers)]
        self._seen_pending = [0 for _ in range(self.layers)]
        self._seen_dev.zero_()
        for group in (self.stored_tokens, self.stored_sinks, self.start_indices, self.pos, self.sink_pos,
                      self.key_cache, self.value_cache, self.score_cache, self.sink_keys, self.sink_values,
                      self.og_pos):
            for t in group:
                t.zero_()
        for group in (self.do_cache, self.mask, self.sink_mask):
            for t in group:
                t.fill_(True)

    def init_cache(self, device):
        """Allocates the state of every layer with the shapes and dtypes of cascading_cache.py:1196-1276."""
        if self.verbose:
            print(f"INIT CLEAN HIP CACHE {self.cascade_func=}")
        n_layers, sinks = self.layers, self.num_sink_tokens
        per_head = (self.max_batch_size, self.heads)
        self._seen_tokens = 0
        self._generation = getattr(self, "_generation", 0) + 1   # recorded graphs and memoised blocks are void
        self._update_memo, self._attn_memo = {}, {}  # argument blocks described once per input layout
        # host mirror of seen_tokens_by_layer: lets callers branch without a device sync
        self._seen_host = [0] * n_layers
        self._seen_pending = [0] * n_layers   # tokens the device counter has not been told about yet
        self.beta = 0.9999999  # cascading_cache.py:1247

        def per_layer(fill, dtype, *tail):
            """One tensor per layer, (batch, heads, *tail(layer)), every element ``fill``."""
            return [torch.full(per_head + tuple(t(l) if callable(t) else t for t in tail), fill, device=device,
                               dtype=dtype) for l in range(n_layers)]

        slots = lambda l: self.max_seq_len[l]    # noqa: E731
        levels = lambda l: self.cascades[l]      # noqa: E731
        self._seen_dev = torch.zeros(n_layers, dtype=torch.long, device=device)
        self.do_cache = [torch.ones(self.cascades[l], device=device, dtype=torch.bool) for l in range(n_layers)]
        self.do_cache_every_n = [
            torch.tensor(acceptance_periods(self.cascade_func, self.cascades[l]), device=device, dtype=torch.long)
            for l in range(n_layers)]
        # trackers and position ids (int64), keys / values / scores (cache dtype), masks (True = empty)
        self.stored_tokens = per_layer(0, torch.long, levels)
        self.start_indices = per_layer(0, torch.long, levels)
        self.stored_sinks = per_layer(0, torch.long)
        self.pos = per_layer(0, torch.long, slots)
        self.og_pos = per_layer(0, torch.long, slots)
        self.sink_pos = per_layer(0, torch.long, sinks)
        self.key_cache = per_layer(0, self.dtype, slots, self.dim)
        self.value_cache = per_layer(0, self.dtype, slots, self.dim)
        self.score_cache = per_layer(0, self.dtype, slots)
        self.sink_keys = per_layer(0, self.dtype, sinks, self.dim)
        self.sink_values = per_layer(0, self.dtype, sinks, self.dim)
        self.mask = per_layer(True, torch.bool, slots)
        self.sink_mask = per_layer(True, torch.bool, sinks)

    @property
    def seen_tokens_by_layer(self) -> Tensor:
        """Tokens seen per layer, on the device (cascading_cache.py:1231); current whenever it is looked at."""
        self._flush_counter()
        return self._seen_dev

    @seen_tokens_by_layer.setter
    def seen_tokens_by_layer(self, value: Tensor):
        self._seen_pending = [0] * self.layers
        self._seen_dev = value

    def _flush_counter(self):
        """Tells the device counter about the updates that went by the constant table."""
        for l, n in enumerate(self._seen_pending):
            if n:
                self._seen_dev[l] += n
                self._seen_pending[l] = 0

    def sync_host_counter(self) -> List[int]:
        """Re-reads the host mirror of ``seen_tokens_by_layer`` from the device (one read-back).

        The fused operator never reads the device counter: the sink shift, the chunk's position ids on an
        eagerly filled cache and the bound on filled slots all come from the host mirror, which ``update`` /
        ``update_state`` / ``reset`` keep in step.  Code that changes the state some other way (copies saved state
        tensors into the cache, calls the module-level ``sink_cache`` and bumps ``seen_tokens_by_layer`` itself, as
        the reference allows) must call this afterwards.  Setting the environment variable ``CKV_DEBUG_COUNTERS=1``
        makes every fused call check the mirror against the device (a device read-back per call)."""
        self._seen_host = [int(x) for x in self.seen_tokens_by_layer.tolist()]
        self._seen_tokens = self._seen_host[0] if self._seen_host else 0
        return list(self._seen_host)

    def check_host_counter(self, layer_idx: int):
        """Raises if the host mirror of a layer's token counter disagrees with the device (a read-back)."""
        dev = int(self.seen_tokens_by_layer[layer_idx])
        if dev != self._seen_host[layer_idx]:
            raise _abi.CkvError(
                f"layer {layer_idx}: the device counter says {dev} tokens, the host mirror {self._seen_host[layer_idx]}; "
                "state was changed outside update()/reset(): call sync_host_counter()")

    def pos_shift(self, layer_idx: int) -> int:
        """The sink shift of get_vals (cascading_cache.py:1282-1283), from the host counter."""
        return self.num_sink_tokens if self._seen_host[layer_idx] > self.num_sink_tokens else 0

    def get_vals(self, layer_idx: int):
        pos_shift = self.pos_shift(layer_idx)
        return (
            self.sink_keys[layer_idx],
            self.sink_values[layer_idx],
            self.sink_pos[layer_idx][:1, 0],
            self.sink_mask[layer_idx],
            self.key_cache[layer_idx],
            self.value_cache[layer_idx],
            self.pos[layer_idx][:1, 0] + pos_shift,
            self.mask[layer_idx],
            self.og_pos[layer_idx],
        )

    def _state_key(self, L: int):
        """Where the layer's state tensors live and how they are laid out: a memoised argument block holds
        raw device pointers and strides, so it is reused only while every state tensor is still at the address
        it was described from.  (Object identity would not do: callers may assign a new tensor to
        ``score_cache[l]`` every step, as cascade_attention.py:222-224 does, and a freed object's id is
        handed out again.)"""
        ts = (self.key_cache[L], self.value_cache[L], self.score_cache[L], self.sink_keys[L], self.sink_values[L],
              self.mask[L], self.sink_mask[L], self.pos[L], self.og_pos[L], self.sink_pos[L], self.stored_tokens[L],
              self.start_indices[L], self.stored_sinks[L], self.do_cache_every_n[L], self._seen_dev)
        return tuple(t.data_ptr() for t in ts) + (self.score_cache[L].stride(), self.score_cache[L].dtype)

    def update(self, key_states: Tensor, value_states: Tensor, layer_idx: int, score_states: Tensor = None):
        """cascading_cache.py:1297-1348."""
        self.update_state(key_states, value_states, layer_idx, score_states)
        return self.get_vals(layer_idx)

    def _update_args(self, key_states: Tensor, value_states: Tensor, score_states: Tensor, L: int):
        """The ``ckv_update`` argument block for these inputs: described once per layer, input layout and
        placement of the state tensors, then reused with only the three input pointers refreshed."""
        key = (L, key_states.shape, key_states.stride(), value_states.shape, value_states.stride(),
               score_states.shape, score_states.stride(), key_states.dtype, value_states.dtype, score_states.dtype,
               key_states.device, value_states.device, score_states.device, self._state_key(L))
        memo = self._update_memo
        a = memo.get(key)
        if a is None:
            a = _abi.fill_update_args(
                key_states, value_states, score_states,
                self.sink_keys[L], self.sink_values[L], self.sink_mask[L], self.sink_pos[L],
                self.key_cache[L], self.value_cache[L], self.score_cache[L],
                self.mask[L], self.pos[L], self.og_pos[L], self.do_cache_every_n[L],
                self.stored_tokens[L], self.start_indices[L], self.stored_sinks[L],
                self.num_sink_tokens, self.window_length[L], self._seen_dev[L], self.max_seq_len[L],
                self.eager_fill)
            a._counter = a.real_token_idx   # the layer's element of the device counter
            a._need = _abi.lib().ckv_update_workspace_bytes(a.N, a.H, a.K, a.max_seq_len, a.cascades)
            if len(memo) > 64:
                memo.clear()
            memo[key] = a
        else:
            a.k, a.v, a.s = key_states.data_ptr(), value_states.data_ptr(), score_states.data_ptr()
        return a

    def update_state(self, key_states: Tensor, value_states: Tensor, layer_idx: int, score_states: Tensor = None,
                     _stream: Optional[int] = None, _device_counter: bool = False):
        """``update`` without building the tuple of views it returns (the shifted position row of
        ``get_vals`` is a device operation of its own); for callers that read the state in place.

        The argument block of ``ckv_update`` is described once per layer and input layout and reused:
        between two calls of the same shape only the three input pointers change (single-token steps
        at batch 1 are bound by this host code, not by the device).  ``_stream``: raw stream handle when
        the caller already holds the device context.

        The update reads the number of tokens seen so far from device memory (``real_token_idx``).  The host knows
        that number, so the call points the library at the element of a constant table ``0, 1, 2, ...`` that holds
        it and leaves the device counter ``seen_tokens_by_layer`` to be brought up to date when somebody looks at
        it: a step then carries no launch for the counter.  ``_device_counter``: read and advance the device counter
        itself, as the reference does (cascading_cache.py:1343-1346): what a step recorded into a graph needs."""
        _require_device(key_states, "k")
        if score_states is None:
            score_states = torch.zeros(self.max_batch_size, self.heads, key_states.size(2),
                                       device=key_states.device, dtype=key_states.dtype)
        if layer_idx == 0:
            self._seen_tokens += key_states.shape[-2]

        a = self._update_args(key_states, value_states, score_states, layer_idx)
        n_new = key_states.shape[-2]
        table = None if _device_counter else _counter_table(key_states.device)
        if table is not None and self._seen_host[layer_idx] < table.numel():
            a.real_token_idx = table.data_ptr() + 8 * self._seen_host[layer_idx]
        else:
            table = None
            self._flush_counter()
            a.real_token_idx = a._counter
        if _stream is None:
            with torch.cuda.device(key_states.device):
                stream = torch.cuda.current_stream(key_states.device).cuda_stream
                ws = workspace(key_states.device, a._need, stream)
                a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
                _abi.check(_abi.lib().ckv_update(C.byref(a), C.c_void_p(stream)), "ckv_update")
        else:
            ws = workspace(key_states.device, a._need, _stream)
            a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
            _abi.check(_abi.lib().ckv_update(C.byref(a), C.c_void_p(_stream)), "ckv_update")
        # after the kernel, as in the reference (cascading_cache.py:1343-1346)
        if table is None:
            self._seen_dev[layer_idx] += n_new
        else:
            self._seen_pending[layer_idx] += n_new
        self._seen_host[layer_idx] += n_new
