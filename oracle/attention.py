"""TEST INFRASTRUCTURE: CPU oracle of the cascade attention path, restated op-for-op in torch.

Follows the reference's eager path so that rounding happens at the same points:
  forward_cascade prologue (positions, RoPE, GQA)  cascade/models/cascade_attention.py:103-200
  cascade_attn_eager                                cascade/models/cascade_attention.py:250-340
  calc_scores                                       cascade/models/cascade_attention.py:231-248
  apply_rotary_pos_emb_one / Llama rope             cascade/models/cascade_attention.py:31-35, 343-352
  rotary cos/sin, rotate_half, repeat_kv            cascade/models/llama/modeling_llama.py:199-220,
                                                    248-252, 316-325

Pinned by tests/test_oracle_attention.py: dense masked softmax attention over the valid keys
(the oracle of cascade/models/test.py:196-219), plain causal attention for an empty cache,
"chunked with cache == dense single shot" when the stream fits one cascade
(cascade/models/test.py:123-165), dense attention with per-head positions for the original-position
mode (cascade_attention.py:141-144, 161-164), the closed forms of the score sums, and torch's own
mean/amax/median for the head reduction.  The bf16 rounding ORDER is not pinned by any
reference test (parity unpinned for that aspect); it is fixed here by using the same torch ops.
"""
import math

import numpy as np
import torch

from .update import OracleCache


def rotary_cos_sin(position_ids, dim, theta, dtype, inv_freq=None):
    """modeling_llama.py:199-220 with the default (unscaled) frequencies."""
    if inv_freq is None:
        inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))
    inv_freq_expanded = inv_freq[None, :, None].float().expand(position_ids.shape[0], -1, 1)
    position_ids_expanded = position_ids[:, None, :].float()
    freqs = (inv_freq_expanded.float() @ position_ids_expanded.float()).transpose(1, 2)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype=dtype), emb.sin().to(dtype=dtype)


def rotate_half(x):
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rope(x, cos, sin):
    """cascade_attention.py:31-35."""
    return (x * cos.unsqueeze(1)) + (rotate_half(x) * sin.unsqueeze(1))


def repeat_kv(x, n_rep):
    b, h, s, d = x.shape
    if n_rep == 1:
        return x
    return x[:, :, None, :, :].expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


_REDUCERS = {
    "mean": torch.mean,
    "max": torch.amax,
    "median": lambda x, **kw: torch.median(x, **kw).values,
}


def calc_scores(scores, homogeneous_heads, n_keys, q_len, kvh, head_reduction):
    """cascade_attention.py:231-248."""
    func = _REDUCERS[head_reduction]
    if homogeneous_heads:
        ema_scores = func(scores[:, :, :n_keys], dim=1, keepdim=True)
        scores = func(scores[:, :, -q_len:], dim=1, keepdim=True).repeat(1, kvh, 1)
    else:
        b, h, s = scores.size()
        ema_scores = func(scores[:, :, :n_keys].view(b, kvh, h // kvh, -1), dim=2)
        scores = func(scores[:, :, -q_len:].view(b, kvh, h // kvh, -1), dim=2)
    return ema_scores, scores


class OracleCascadeAttention:
    """One attention layer over an :class:`OracleCache` (projections excluded)."""

    def __init__(self, num_heads, num_kv_heads, head_dim, rope_theta=500000.0, head_reduction="mean",
                 homogeneous_heads=False, do_og_pos=False):
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.groups = num_heads // num_kv_heads
        self.rope_theta = rope_theta
        self.head_reduction = head_reduction
        self.homogeneous_heads = homogeneous_heads
        self.do_og_pos = do_og_pos  # cached keys rotated per (batch, head) at their original token index
        self.last_q_size = None
        self.query_pos = None
        self.causal_mask = None
        self.ema_mask = None

    def rope(self, x, pos):
        cos, sin = rotary_cos_sin(pos, self.head_dim, self.rope_theta, x.dtype)
        return apply_rope(x, cos, sin)

    def forward(self, query_states, key_states, value_states, cache: OracleCache, return_probs=False):
        """query (B,H,q,D), key/value (B,KVH,q,D), all un-rotated.  Returns out (B,H,q,D) and
        mutates the cache exactly like forward_cascade + cascade_attn_eager."""
        q_len = query_states.size(2)
        first_it = int(cache.seen_tokens) == 0  # cascade_attention.py:114

        sink_k, sink_v, sink_pos, sink_mask, k_states, v_states, key_pos, key_mask, og_pos = cache.get_vals()

        max_pos = 0
        if first_it:  # cascade_attention.py:120-123
            self.query_pos = torch.arange(0, q_len, dtype=torch.long).view(1, -1)
        elif self.do_og_pos:  # cascade_attention.py:141-144
            max_pos = torch.cat((sink_pos.amax().view(1), og_pos.amax().view(1)), dim=-1).amax() + 1
        else:  # cascade_attention.py:145-148
            max_pos = torch.cat((sink_pos.amax().view(1), key_pos.amax().view(1)), dim=-1).amax() + 1
        query_pos = self.query_pos[:, :q_len] + max_pos  # cascade_attention.py:150

        # cascade_attention.py:157-166
        query_states = self.rope(query_states, query_pos)
        key_states_pos = self.rope(key_states, query_pos)
        sink_k = self.rope(sink_k, sink_pos)
        if self.do_og_pos:  # cascade_attention.py:161-164
            b, h, s, d = k_states.size()
            k_states = self.rope(k_states.view(b * h, 1, s, d), og_pos.view(b * h, -1)).view(b, h, s, d)
        else:
            k_states = self.rope(k_states, key_pos)

        g = self.groups
        key_states_pos = repeat_kv(key_states_pos, g)
        sink_k = repeat_kv(sink_k, g)
        sink_v = repeat_kv(sink_v, g)
        k_states = repeat_kv(k_states, g)
        v_states = repeat_kv(v_states, g)
        scale = 1 / math.sqrt(query_states.size(-1))

        # ---- cascade_attn_eager, cascade_attention.py:258-340 ----
        dtype = query_states.dtype
        val = torch.finfo(dtype).min
        if first_it or self.last_q_size != q_len:
            self.last_q_size = q_len
            self.causal_mask = torch.full((q_len, q_len), True, dtype=torch.bool).triu(1)
            beta = cache.beta
            # column n of the reference's mask holds (1-beta)*beta**arange(q_len-n) below the
            # diagonal (cascade_attention.py:270-282); every column is a prefix of one vector
            e = (1 - beta) * beta ** torch.arange(q_len, dtype=dtype)
            idx = torch.arange(q_len)[:, None] - torch.arange(q_len)[None, :]
            self.ema_mask = torch.where(idx >= 0, e[idx.clamp(min=0)], torch.zeros((), dtype=dtype))

        rs = np.sqrt(scale)
        qattn = torch.einsum("bhqd,bhkd->bhqk", query_states * rs, key_states_pos * rs)
        qattn = qattn + (self.causal_mask * val).to(qattn.dtype)
        sattn = torch.einsum("bhqd,bhkd->bhqk", query_states * rs, sink_k * rs)
        sattn = sattn + (val * sink_mask[:1, :1, None, :]).to(qattn.dtype)
        cattn = torch.einsum("bhqd,bhkd->bhqk", query_states * rs, k_states * rs)
        cattn = cattn + (val * key_mask[:1, :1, None, :]).to(qattn.dtype)

        attn = torch.cat((sattn, cattn, qattn), dim=-1)
        attn = attn.softmax(dim=-1)

        sk, k = sink_k.size(2), k_states.size(2)
        out = attn[:, :, :, :sk] @ sink_v
        out += attn[:, :, :, sk:sk + k] @ v_states
        out += attn[:, :, :, -q_len:] @ repeat_kv(value_states, g)

        beta = cache.beta
        exps = (1 - beta) * beta ** torch.arange(attn.size(2)).flip(dims=(0,))
        ema_scores = (attn[:, :, :, sk:sk + k] * exps[None, None, :, None]).sum(dim=2).to(attn.dtype)

        scores = attn[:, :, :, -q_len:] * self.ema_mask[None, None, :].to(attn.dtype)
        scores = scores.sum(dim=2)
        scores = torch.cat((ema_scores, scores), dim=-1)

        ema_scores, scores = calc_scores(scores, self.homogeneous_heads, k, q_len, self.num_kv_heads,
                                         self.head_reduction)
        cache.score_cache = beta ** scores.size(2) * cache.score_cache + ema_scores
        if cache.score_cache.dtype != dtype:
            cache.score_cache = cache.score_cache.to(dtype)
        scores = scores.repeat(1, query_states.size(1), 1)
        self.last_new_scores = scores
        self.last_ema = ema_scores
        self.last_score_cache = cache.score_cache.clone()  # what the update's evictions will carry

        cache.update(key_states, value_states, score_states=scores)
        if return_probs:
            return out, attn
        return out
