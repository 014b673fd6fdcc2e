"""Host-side mirror of the reference's attention wrapper (cascade/models/cascade_attention.py).

``cascade_attention`` is the fused operator: one ``ckv_attn`` call replaces the RoPE of the whole
cache, ``repeat_kv``, the concatenations, ``attention``/the eager matmuls, ``calc_scores`` and the
score-EMA assignment (cascade_attention.py:150-224 / 250-330), then ``cache.update`` scatters the
chunk (cascade_attention.py:226-227, 334-339).  ``CascadeAttention`` keeps the method names of
the reference mixin so model code written against it keeps working.
"""
import ctypes as C
import math
import os
from typing import Optional

import torch
from torch import nn

from . import _abi
from .cascading_cache import CascadingKVCache, _require_device, workspace


_DEBUG_COUNTERS = os.environ.get("CKV_DEBUG_COUNTERS", "0") not in ("", "0")


def default_inv_freq(head_dim: int, theta: float, device) -> torch.Tensor:
    """The unscaled rotary frequencies, computed exactly like the HF default initialiser the
    reference model uses (modeling_llama.py:166-177): fp32 ``1 / theta^(2i/d)``."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    return inv.to(device)


def chunk_positions(cache: CascadingKVCache, layer_idx: int, q_len: int, do_og_pos: bool = False,
                    _stream: Optional[int] = None, _replayable: bool = False) -> torch.Tensor:
    """Position ids of the incoming chunk (cascade_attention.py:119-150) without a host sync:
    0.. on the first call, otherwise one past the largest id among sinks and cache slots
    (stale and masked entries included, as in the reference).  One small kernel of the library.
    ``_stream``: raw stream handle when the caller already holds the device context."""
    _require_device(cache.key_cache[layer_idx], "the cache")
    dev = cache.key_cache[layer_idx].device
    # An eagerly filled cache drops no token before it is full: every token up to index S + num_sink is accepted by
    # every cascade (cascading_cache.py:471-478), so sinks and slots together hold min(seen, S + num_sink) tokens,
    # their ids are 0 .. that - 1 (stale entries of slots not yet filled are never larger: the position pass hands
    # out ids below the number of stored tokens, cascading_cache.py:112-142), and the chunk starts one past them
    # whatever the stream does later.  The ids are then a function of the host-side token counter: no kernel, no
    # device read.  (This holds for every state the update itself produces from an empty cache.)
    # A caller that records the launches for replay always gets the ids from the device: a recorded launch keeps
    # the raw pointer of this tensor, which must neither depend on the host counter nor be freed under it.
    S, NS = cache.max_seq_len[layer_idx], cache.num_sink_tokens
    if not do_og_pos and cache.eager_fill and S > 0 and not _replayable:
        start = min(int(cache._seen_host[layer_idx]), S + NS)
        memo = cache.__dict__.setdefault("_steady_q_pos", {})
        key = (start, q_len, dev)
        ids = memo.get(key)
        if ids is None:
            if len(memo) > 16:
                memo.clear()
            ids = memo[key] = torch.arange(start, start + q_len, device=dev, dtype=torch.long)
        return ids
    out = torch.empty(q_len, device=dev, dtype=torch.long)
    key_ptr, n_key, shift, sink_ptr, n_sink = None, 0, 0, None, 0
    if cache._seen_host[layer_idx] != 0:
        if do_og_pos:
            og = cache.og_pos[layer_idx]
            assert og.is_contiguous()
            key_ptr, n_key = og.data_ptr(), og.numel()
        else:
            row = cache.pos[layer_idx][0, 0]
            assert row.is_contiguous()
            key_ptr, n_key, shift = row.data_ptr(), row.numel(), int(cache.pos_shift(layer_idx))
        if cache.num_sink_tokens > 0:
            srow = cache.sink_pos[layer_idx][0, 0]
            assert srow.is_contiguous()
            sink_ptr, n_sink = srow.data_ptr(), srow.numel()
    if _stream is None:
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            _abi.check(_abi.lib().ckv_chunk_positions(key_ptr, n_key, shift, sink_ptr, n_sink, q_len, out.data_ptr(), stream),
                       "ckv_chunk_positions")
    else:
        _abi.check(_abi.lib().ckv_chunk_positions(key_ptr, n_key, shift, sink_ptr, n_sink, q_len, out.data_ptr(), _stream),
                   "ckv_chunk_positions")
    return out


def check_against_cache(query_states, key_states, value_states, cache: CascadingKVCache, L: int):
    """The kernels index the cache tensors with the sizes of the incoming chunk, so every size the two
    share is checked here, on the host, before any pointer leaves: a mismatch raises instead of reading
    or writing past the cache allocations (the reference fails with a torch shape or dtype error at its
    ``torch.cat`` / ``einsum`` calls, cascade_attention.py:212-218, 284-291)."""
    B, H, Q, D = query_states.shape
    KVH = key_states.size(1)
    if not 0 <= L < cache.layers:
        raise ValueError(f"layer {L} outside the cache's {cache.layers} layers")
    kc = cache.key_cache[L]
    if H % KVH != 0:
        raise ValueError(f"{H} query heads are not a multiple of {KVH} kv heads")
    if B > kc.size(0):
        raise ValueError(f"batch {B} exceeds the cache's max_batch_size {kc.size(0)}")
    if KVH != kc.size(1):
        raise ValueError(f"{KVH} kv heads, but the cache holds {kc.size(1)}")
    if D != kc.size(3):
        raise ValueError(f"head_dim {D}, but the cache holds rows of {kc.size(3)}")
    for name, t in (("query_states", query_states), ("key_states", key_states), ("value_states", value_states)):
        if t.dtype != kc.dtype:
            raise TypeError(f"{name} is {t.dtype}, the cache is {kc.dtype}")
        if t.device != kc.device:
            raise ValueError(f"{name} lives on {t.device}, the cache on {kc.device}")


def _describe_attention(query_states, key_states, value_states, cache, L, inv_freq, reduction, homogeneous_heads,
                        do_og_pos, scale, out, new_scores):
    """The argument block of ``ckv_attn`` for one layer and input layout; everything in it except the
    pointers of the per-call tensors and the sink shift stays valid from call to call."""
    lib = _abi.lib()
    B, H, Q, D = query_states.shape
    KVH = key_states.size(1)
    NS, S = cache.num_sink_tokens, cache.max_seq_len[L]
    a = _abi.AttnArgs()
    _abi.set_strides(a.q_stride, query_states)
    _abi.set_strides(a.kv_new_stride, key_states)
    a.sink_k, a.sink_v = cache.sink_keys[L].data_ptr(), cache.sink_values[L].data_ptr()
    _abi.set_strides(a.sink_stride, cache.sink_keys[L])
    a.cache_k, a.cache_v = cache.key_cache[L].data_ptr(), cache.value_cache[L].data_ptr()
    _abi.set_strides(a.cache_stride, cache.key_cache[L])
    assert cache.sink_mask[L].stride(-1) == 1 and cache.mask[L].stride(-1) == 1
    a.sink_mask, a.mask = cache.sink_mask[L].data_ptr(), cache.mask[L].data_ptr()  # row [0, 0]
    assert cache.sink_pos[L].stride(-1) == 1 and cache.pos[L].stride(-1) == 1 and cache.og_pos[L].stride(-1) == 1
    a.sink_pos = cache.sink_pos[L].data_ptr()
    a.sink_pos_stride[0], a.sink_pos_stride[1] = 0, 0
    if do_og_pos:  # every (batch, head) rotates its keys at their original positions (:161-164)
        a.pos = cache.og_pos[L].data_ptr()
        a.pos_stride[0], a.pos_stride[1] = cache.og_pos[L].stride(0), cache.og_pos[L].stride(1)
    else:
        a.pos = cache.pos[L].data_ptr()
        a.pos_stride[0], a.pos_stride[1] = 0, 0
    a.cache_s = cache.score_cache[L].data_ptr()
    _abi.set_strides(a.cache_s_stride, cache.score_cache[L])
    _abi.set_strides(a.out_stride, out)
    _abi.set_strides(a.new_scores_stride, new_scores)
    a.lse = None
    a.B, a.H, a.KVH, a.Q, a.D = B, H, KVH, Q, D
    a.num_sink, a.S = NS, S
    a.scale = float(scale)
    a.rope_theta = 0.0
    assert inv_freq.dtype == torch.float32 and inv_freq.numel() == D // 2 and inv_freq.is_contiguous()
    a.inv_freq = inv_freq.data_ptr()
    a.beta = float(cache.beta)
    a.head_reduction = _abi.CKV_REDUCE[reduction]
    a.homogeneous_heads = int(bool(homogeneous_heads))
    a.dtype = _abi.dtype_code(query_states.dtype)
    a._need = lib.ckv_attn_workspace_bytes(B, H, KVH, Q, D, NS, S, a.dtype)
    return a


def cascade_attention(query_states, key_states, value_states, cache: CascadingKVCache, layer_idx: int,
                      inv_freq: torch.Tensor, head_reduction: Optional[str] = None,
                      homogeneous_heads: bool = False, do_og_pos: bool = False, scale: Optional[float] = None,
                      update_cache: bool = True, replayable: bool = False):
    """Attention of one chunk over [sink | cascades | chunk] plus the cache bookkeeping.

    query_states ``(B, H, q, D)``, key/value_states ``(B, KVH, q, D)``, all un-rotated.
    Returns ``out (B, H, q, D)``; mutates ``cache.score_cache[layer_idx]`` and, if
    ``update_cache``, scatters the chunk into the cache with its new scores.
    ``replayable``: the launches are being recorded for replay (a HIP graph), so nothing that the host derives
    from its token counter and that changes from call to call may go into them: position ids come from the device
    unless the cache is full, and the library is not told how many slots are filled.
    """
    _require_device(query_states, "query_states")
    lib = _abi.lib()
    if _DEBUG_COUNTERS:
        cache.check_host_counter(layer_idx)
    B, H, Q, D = query_states.shape
    KVH = key_states.size(1)
    assert key_states.shape == (B, KVH, Q, D) and value_states.shape == (B, KVH, Q, D)
    assert _abi.same_layout(key_states, value_states)
    dtype = query_states.dtype
    dev = query_states.device
    L = layer_idx
    reduction = head_reduction or cache.head_reduction
    if scale is None:
        scale = 1 / math.sqrt(D)

    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        q_pos = chunk_positions(cache, L, Q, do_og_pos, _stream=stream, _replayable=replayable)
        out = torch.empty((B, H, Q, D), dtype=dtype, device=dev)
        new_scores = torch.empty((B, KVH, Q), dtype=dtype, device=dev)

        # the argument block is described once per layer and input layout (single-token steps at batch 1
        # are bound by this host code, not by the device)
        key = (L, query_states.shape, query_states.stride(), key_states.shape, key_states.stride(), dtype,
               key_states.dtype, value_states.dtype, dev, key_states.device, value_states.device, reduction,
               bool(homogeneous_heads), bool(do_og_pos), float(scale), float(cache.beta), inv_freq.data_ptr(),
               inv_freq.dtype, cache._state_key(L))
        a = cache._attn_memo.get(key)
        if a is None:  # a layout not seen before: validated once, then described
            check_against_cache(query_states, key_states, value_states, cache, L)
            a = _describe_attention(query_states, key_states, value_states, cache, L, inv_freq, reduction,
                                    homogeneous_heads, do_og_pos, scale, out, new_scores)
            if len(cache._attn_memo) > 64:
                cache._attn_memo.clear()
            cache._attn_memo[key] = a
        a.q = query_states.data_ptr()
        a.k_new, a.v_new = key_states.data_ptr(), value_states.data_ptr()
        a.q_pos = q_pos.data_ptr()
        a.pos_shift = 0 if do_og_pos else cache.pos_shift(L)
        # the cache fills from slot 0 up and holds at most the tokens seen past the sinks: single-token steps skip
        # the empty part of a cache that is still filling
        filled = int(cache._seen_host[L]) - cache.num_sink_tokens
        a.filled_slots = filled if not replayable and 0 < filled < cache.max_seq_len[L] else 0
        a.out = out.data_ptr()
        a.new_scores = new_scores.data_ptr()
        ws = workspace(dev, a._need, stream)
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
        _abi.check(lib.ckv_attn(C.byref(a), C.c_void_p(stream)), "ckv_attn")
        if update_cache:
            cache.update_state(key_states, value_states, L, score_states=new_scores, _stream=stream,
                               _device_counter=replayable)
    return out, new_scores


class DecodeStepGraph:
    """Single-token steps of one layer replayed from a HIP graph.

    A decode step is a chain of short kernels (query rotation, streaming attention, combine, scores, update plan,
    update apply, the token counter); at batch 1 and small windows the host needs longer to launch them than the
    device to run them.  The first ``step`` runs eagerly (it sets kernel attributes and sizes the scratch), the
    second one records the same calls into a graph, and every later one copies the token's q, k, v into the
    graph's fixed input buffers and replays it.  The cache is advanced exactly as by ``cascade_attention``; the
    returned ``out`` / ``new_scores`` tensors are the graph's fixed outputs and are overwritten by the next step.

    Recorded values that must not change between steps: the sink shift (the cache must already hold more than
    ``num_sink_tokens`` tokens), shapes, dtype, head reduction, and the addresses of the cache's state tensors
    (assigning a new tensor to ``score_cache[l]`` raises at the next step: build a new graph).  The position ids of
    the token come from a kernel inside the graph, never from the host counter.  ``reset()`` / ``init_cache()`` of
    the cache are noticed (the cache counts them): the next step runs eagerly and the one after records afresh."""

    def __init__(self, cache: CascadingKVCache, layer_idx: int, inv_freq: torch.Tensor, num_heads: int,
                 head_reduction: Optional[str] = None, homogeneous_heads: bool = False, do_og_pos: bool = False,
                 scale: Optional[float] = None):
        self.cache, self.layer_idx, self.inv_freq = cache, layer_idx, inv_freq
        self.kw = dict(head_reduction=head_reduction, homogeneous_heads=homogeneous_heads, do_og_pos=do_og_pos,
                       scale=scale)
        kc = cache.key_cache[layer_idx]
        B, KVH, _, D = kc.shape
        self.q = torch.empty(B, num_heads, 1, D, dtype=kc.dtype, device=kc.device)
        self.k = torch.empty(B, KVH, 1, D, dtype=kc.dtype, device=kc.device)
        self.v = torch.empty(B, KVH, 1, D, dtype=kc.dtype, device=kc.device)
        self.graph = None
        self.out = self.new_scores = None
        self._warm = False
        self._state = None
        self._generation = None

    def _run(self):
        return cascade_attention(self.q, self.k, self.v, self.cache, self.layer_idx, self.inv_freq, replayable=True,
                                 **self.kw)

    def step(self, q=None, k=None, v=None):
        """One token: ``q (B, H, 1, D)``, ``k, v (B, KVH, 1, D)`` (or None when the caller has written them into
        ``self.q / self.k / self.v`` already).  Returns ``(out, new_scores)``."""
        cache, L = self.cache, self.layer_idx
        if cache._seen_host[L] <= cache.num_sink_tokens:
            raise _abi.CkvError("DecodeStepGraph needs a cache that already holds more than num_sink_tokens tokens")
        if q is not None:
            self.q.copy_(q)
            self.k.copy_(k)
            self.v.copy_(v)
        cache._flush_counter()  # the recorded update reads and advances the device counter itself
        if self._generation != cache._generation:  # first use, or the cache was reset / reallocated since
            self._generation = cache._generation
            self.graph, self._warm = None, False
        if not self._warm:  # eager: kernel attributes, scratch sizes, argument blocks
            self._warm = True
            return self._run()
        if self.graph is not None and self._state != cache._state_key(L):
            raise _abi.CkvError("the cache's state tensors moved since the graph was recorded")
        if self.graph is None:
            if _abi.profile_enable(0) != 0:
                raise _abi.CkvError("stage timing must be off while a step is recorded")
            seen_host, seen_total = cache._seen_host[L], cache._seen_tokens
            self._state = cache._state_key(L)
            torch.cuda.synchronize(self.q.device)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.out, self.new_scores = self._run()
            # recording ran no kernel: only the host-side counters moved, and the replay below is the step
            cache._seen_host[L], cache._seen_tokens = seen_host, seen_total
        self.graph.replay()
        cache._seen_host[L] += 1
        if L == 0:
            cache._seen_tokens += 1
        return self.out, self.new_scores


def _rotate(x, cos, sin):
    """``x * cos + rotate_half(x) * sin`` in ``x.dtype``, cos / sin ``(B or 1, n, D)`` broadcast over heads."""
    half = x.size(-1) // 2
    turned = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return x * cos[:, None] + turned * sin[:, None]


class CascadeAttention(nn.Module):
    """Attention layer with the reference mixin's surface (cascade_attention.py:38-340).

    A concrete layer provides ``q_proj/k_proj/v_proj/o_proj``, ``num_heads``,
    ``num_key_value_heads``, ``head_dim``, ``layer_idx``, ``rope_theta`` and a ``config`` with
    ``_homogeneous_heads``, ``_do_og_pos`` and ``_head_reduction`` (llama_eval.py:142-152).
    Chunked prefill and single-token decode both run the fused HIP path; there is no eager arm.
    """

    def forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_value=None,
                output_attentions=False, use_cache=False, cache_position=None, position_embeddings=None):
        if isinstance(past_key_value, CascadingKVCache):
            return self.forward_cascade(
                hidden_states=hidden_states, past_key_value=past_key_value,
                homogeneous_heads=self.config._homogeneous_heads, do_og_pos=self.config._do_og_pos)
        raise ValueError("unknown custom attention")

    def qkv(self, x, size, kv_size):
        """Projections reshaped to (batch, heads, tokens, head_dim) (cascade_attention.py:74-80)."""
        return (self.q_proj(x).view(*size).transpose(1, 2), self.k_proj(x).view(*kv_size).transpose(1, 2),
                self.v_proj(x).view(*kv_size).transpose(1, 2))

    def forward_cascade(self, hidden_states, attention_mask=None, position_ids=None, past_key_value=None,
                        output_attentions=False, use_cache=False, cache_position=None, use_flash=True,
                        homogeneous_heads=True, do_og_pos=False, use_selfextend=False, position_embeddings=None):
        if use_selfextend:
            raise NotImplementedError("use_selfextend is a dead arm in the reference (never enabled)")
        bsz, q_len, _ = hidden_states.size()
        query_states, key_states, value_states = self.qkv(
            hidden_states, (bsz, q_len, self.num_heads, self.head_dim),
            (bsz, q_len, self.num_key_value_heads, self.head_dim))
        if not hasattr(self, "_inv_freq") or self._inv_freq.device != hidden_states.device:
            self._inv_freq = default_inv_freq(self.head_dim, self.rope_theta, hidden_states.device)
        out, _ = cascade_attention(query_states, key_states, value_states, past_key_value, self.layer_idx,
                                   self._inv_freq, head_reduction=self.config._head_reduction,
                                   homogeneous_heads=homogeneous_heads, do_og_pos=do_og_pos)
        out = out.transpose(1, 2).contiguous().view(bsz, q_len, -1)
        out = self.o_proj(out)
        return out, None, past_key_value

    # -- the reference mixin's remaining surface -------------------------------------------------------------
    # ``forward_cascade`` above never calls these (the fused operator rotates, concatenates and reduces inside
    # the kernels); they exist so that model code written against the reference mixin, which calls
    # ``self.rope(...)`` and ``self.cascade_attn_flash(...)`` / ``self.cascade_attn_eager(...)`` itself, keeps
    # working.  Both attention arms run the library's dense operator, whose scores are exact.

    def rope(self, x, pos, cos=None, sin=None):
        """Rotary embedding of ``x (B, heads, n, D)`` at positions ``pos (B or 1, n)``; returns
        ``(rotated, cos, sin)`` so the caller can reuse the tables (cascade_attention.py:343-353).  Angles are
        fp32 ``pos * inv_freq``; cos / sin are cast to ``x.dtype`` before they are applied
        (modeling_llama.py:205-220, 248-252)."""
        if cos is None or sin is None:
            if not hasattr(self, "_inv_freq") or self._inv_freq.device != x.device:
                self._inv_freq = default_inv_freq(self.head_dim, self.rope_theta, x.device)
            angles = pos.to(torch.float32)[..., None] * self._inv_freq       # (B, n, D/2)
            angles = torch.cat((angles, angles), dim=-1)
            cos, sin = angles.cos().to(x.dtype), angles.sin().to(x.dtype)
        return _rotate(x, cos, sin), cos, sin

    def cascade_attn_flash(self, query_states, key_states, value_states, key_states_pos, v_states, sink_key_states,
                           sink_value_states, k_states, sink_mask, key_mask, first_it, past_key_value, scale, q_len,
                           homogeneous_heads):
        """cascade_attention.py:202-229 on the library's dense operator: the caller has rotated and head-expanded
        everything except ``key_states`` / ``value_states`` (the chunk as it goes into the cache).  The sums of the
        cached keys are taken aligned with their slots, as the eager arm does (cascade_attention.py:319); the
        reference's flash arm hands ``calc_scores`` the first ``n_keys`` columns, sink columns included."""
        from .flash_attention import attention

        self.last_attn_called, self.last_q_size = "flash", query_states.size(2)
        groups = query_states.size(1) // value_states.size(1)
        chunk_values = value_states[:, :, None].expand(-1, -1, groups, -1, -1).reshape(
            value_states.size(0), -1, value_states.size(2), value_states.size(3))       # repeat_kv
        keys = torch.cat((sink_key_states, k_states, key_states_pos), dim=2)
        values = torch.cat((sink_value_states, v_states, chunk_values), dim=2)
        hidden = torch.cat((sink_mask[0, 0], key_mask[0, 0]))
        out, scores = attention(query_states, keys, values, True, scale, hidden, past_key_value.beta)
        # the dense operator's scores cover [sink | cache | chunk]; the cached part is what the EMA is for
        n_sink = sink_key_states.size(2)
        ema, new_scores = self.calc_scores(scores[:, :, n_sink:], homogeneous_heads, k_states.size(2), q_len)
        L = self.layer_idx
        past_key_value.score_cache[L] = (past_key_value.beta ** q_len) * past_key_value.score_cache[L] + ema
        past_key_value.update(key_states, value_states, L, score_states=new_scores)
        return out, past_key_value

    def cascade_attn_eager(self, *args):
        """cascade_attention.py:250-340.  There is no eager arm on the device: the dense operator already returns
        the exact sums the eager path computes, so this is ``cascade_attn_flash`` under the other name."""
        out, cache = self.cascade_attn_flash(*args)
        self.last_attn_called = "eager"
        return out, cache

    def calc_scores(self, scores, homogeneous_heads, n_keys, q_len):
        """Head reduction of per-head score sums ``(B, H, n)`` with the semantics of
        cascade_attention.py:231-248, for callers that hold per-head scores of their own (``attention``
        returns them); the fused path reduces inside the kernels.  The heads are viewed as
        ``(groups, members)``: one group of all heads when ``homogeneous_heads`` (its result serves every kv
        head), otherwise one group per kv head.  Returns the reduced scores of the first ``n_keys`` keys
        ``(B, groups, n_keys)`` and of the last ``q_len`` keys ``(B, KVH, q_len)``."""
        kvh = self.num_key_value_heads
        b, h, _ = scores.shape
        groups = 1 if homogeneous_heads else kvh
        grouped = scores.view(b, groups, h // groups, -1)
        how = self.config._head_reduction
        if how == "mean":
            reduced = grouped.mean(dim=2)
        elif how == "max":
            reduced = grouped.amax(dim=2)
        elif how == "median":
            reduced = grouped.median(dim=2).values
        else:
            raise KeyError(how)
        new_scores = reduced[:, :, -q_len:]
        if homogeneous_heads:
            new_scores = new_scores.repeat(1, kvh, 1)
        return reduced[:, :, :n_keys], new_scores


class LlamaCascadeAttention(CascadeAttention):
    """cascade_attention.py:343-353: cos / sin computed from the position ids (the mixin's default ``rope``)."""


class Qwen2CascadeAttention(CascadeAttention):
    """cascade_attention.py:356-367: cos / sin looked up in a table of ``max_position_embeddings`` rows (the ids
    of a cascade cache can exceed the length a Qwen2 rotary module was asked for, hence the fixed table)."""

    def rope(self, x, pos, cos=None, sin=None):
        if cos is None or sin is None:
            if not hasattr(self, "_inv_freq") or self._inv_freq.device != x.device:
                self._inv_freq = default_inv_freq(self.head_dim, self.rope_theta, x.device)
            rows = torch.arange(self.max_position_embeddings, device=x.device, dtype=torch.float32)
            angles = torch.outer(rows, self._inv_freq)
            angles = torch.cat((angles, angles), dim=-1)
            cos, sin = angles.cos().to(x.dtype), angles.sin().to(x.dtype)
        ids = pos.reshape(-1)
        picked_cos = cos[ids].reshape(1, pos.size(1), cos.size(-1))
        picked_sin = sin[ids].reshape(1, pos.size(1), sin.size(-1))
        return _rotate(x, picked_cos, picked_sin), cos, sin
