"""Pins the CPU attention oracle (oracle/attention.py) against library routines and closed forms.

Nothing here re-types the oracle's formulas: the dense references use complex-number RoPE,
torch.softmax / scaled_dot_product_attention on explicitly gathered keys, and float64 loops.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle.attention import OracleCascadeAttention, calc_scores
from oracle.update import OracleCache


def rope_complex(x, pos, theta):
    """Textbook rotary embedding: pairs (x[d], x[d + D/2]) rotated by pos * theta^(-2d/D)."""
    D = x.size(-1)
    xd = x.double()
    z = torch.complex(xd[..., : D // 2], xd[..., D // 2:])
    freq = theta ** (-torch.arange(0, D, 2, dtype=torch.float64) / D)
    ang = pos.double()[..., None] * freq
    z = z * torch.polar(torch.ones_like(ang), ang)
    return torch.cat((z.real, z.imag), dim=-1)


def dense_reference(q, k_new, v_new, cache: OracleCache, theta, q_pos):
    """softmax(QK^T/sqrt(D)) V over exactly the keys a query may see, in float64."""
    B, H, Q, D = q.shape
    KVH = k_new.size(1)
    G = H // KVH
    sink_k, sink_v, sink_pos, sink_mask, ck, cv, key_pos, key_mask, _ = cache.get_vals()
    sv = ~sink_mask[0, 0]
    cvalid = ~key_mask[0, 0]
    keys = torch.cat((rope_complex(sink_k[:, :, sv], sink_pos[0, sv], theta),
                      rope_complex(ck[:, :, cvalid], key_pos[0, cvalid], theta),
                      rope_complex(k_new, q_pos, theta)), dim=2)
    vals = torch.cat((sink_v[:, :, sv], cv[:, :, cvalid], v_new), dim=2).double()
    keys = keys.repeat_interleave(G, dim=1)
    vals = vals.repeat_interleave(G, dim=1)
    qr = rope_complex(q, q_pos, theta)
    n_prev = keys.size(2) - Q
    logits = qr @ keys.transpose(-1, -2) / math.sqrt(D)
    causal = torch.ones(Q, Q, dtype=torch.bool).triu(1)
    logits[..., n_prev:] = logits[..., n_prev:].masked_fill(causal, float("-inf"))
    p = torch.softmax(logits, dim=-1)
    return p @ vals, p, n_prev


def make_layer(B=1, H=4, KVH=2, D=16, NS=2, W=8, C=2, eager=True, dtype=torch.float32, reduction="mean",
               homogeneous=False, theta=10000.0):
    cache = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D, max_seq_len=W * C,
                        dtype=dtype, eager_fill=eager)
    attn = OracleCascadeAttention(H, KVH, D, rope_theta=theta, head_reduction=reduction, homogeneous_heads=homogeneous)
    return cache, attn


def rand_chunk(g, B, H, KVH, Q, D, dtype=torch.float32):
    return (torch.randn(B, H, Q, D, generator=g).to(dtype), torch.randn(B, KVH, Q, D, generator=g).to(dtype),
            torch.randn(B, KVH, Q, D, generator=g).to(dtype))


def test_first_chunk_is_plain_causal_attention():
    g = torch.Generator().manual_seed(0)
    cache, attn = make_layer(B=2, H=4, KVH=2, D=16)
    q, k, v = rand_chunk(g, 2, 4, 2, 6, 16)
    out = attn.forward(q, k, v, cache)
    pos = torch.arange(6)
    ref = F.scaled_dot_product_attention(rope_complex(q, pos, 10000.0),
                                         rope_complex(k, pos, 10000.0).repeat_interleave(2, dim=1),
                                         v.double().repeat_interleave(2, dim=1), is_causal=True)
    assert torch.allclose(out.double(), ref, atol=1e-5)


@pytest.mark.parametrize("C,eager", [(1, True), (2, True), (4, False), (2, False)])
def test_every_chunk_matches_dense_attention_over_valid_keys(C, eager):
    g = torch.Generator().manual_seed(1)
    B, H, KVH, D, NS, W, Q = 2, 6, 2, 8, 3, 4, 5
    cache, attn = make_layer(B, H, KVH, D, NS, W, C, eager)
    for step in range(12):
        q, k, v = rand_chunk(g, B, H, KVH, Q, D)
        # positions the chunk must get: one past the largest id handed out by the cache
        if step == 0:
            q_pos = torch.arange(Q)
        else:
            vals = cache.get_vals()
            q_pos = torch.arange(Q) + max(int(vals[2].max()), int(vals[6].max())) + 1
        ref, _, _ = dense_reference(q, k, v, cache, 10000.0, q_pos)
        out = attn.forward(q, k, v, cache)
        assert torch.allclose(out.double(), ref, atol=2e-5), f"chunk {step}"


def test_original_position_mode_matches_dense_attention_with_per_head_positions():
    """cascade_attention.py:141-144, 161-164 (do_og_pos): cached keys are rotated per (batch, head) at the
    1-based index of the token each slot holds, sinks at their slot number, the chunk one past the
    largest index in the cache.  Scores differ per head, so the heads keep different tokens."""
    g = torch.Generator().manual_seed(7)
    B, H, KVH, D, NS, W, C, Q, theta = 2, 4, 2, 8, 2, 4, 2, 3, 10000.0
    cache = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D, max_seq_len=W * C,
                        dtype=torch.float32, eager_fill=False)
    attn = OracleCascadeAttention(H, KVH, D, rope_theta=theta, do_og_pos=True)
    differed = False
    for step in range(14):
        q, k, v = rand_chunk(g, B, H, KVH, Q, D)
        sink_k, sink_v, sink_pos, sink_mask, ck, cv, _key_pos, key_mask, og_pos = cache.get_vals()
        sv, cvalid = ~sink_mask[0, 0], ~key_mask[0, 0]
        differed = differed or not torch.equal(og_pos[0, 0, cvalid], og_pos[0, 1, cvalid])
        q_pos = torch.arange(Q) + (0 if step == 0 else max(int(sink_pos.max()), int(og_pos.max())) + 1)
        keys = torch.cat((rope_complex(sink_k[:, :, sv], sink_pos[0, sv], theta),
                          rope_complex(ck[:, :, cvalid], og_pos[:, :, cvalid], theta),
                          rope_complex(k, q_pos, theta)), dim=2).repeat_interleave(H // KVH, dim=1)
        vals = torch.cat((sink_v[:, :, sv], cv[:, :, cvalid], v), dim=2).double().repeat_interleave(H // KVH, dim=1)
        n_prev = keys.size(2) - Q
        logits = rope_complex(q, q_pos, theta) @ keys.transpose(-1, -2) / math.sqrt(D)
        logits[..., n_prev:] = logits[..., n_prev:].masked_fill(torch.ones(Q, Q, dtype=torch.bool).triu(1), float("-inf"))
        ref = torch.softmax(logits, dim=-1) @ vals
        out = attn.forward(q, k, v, cache)
        assert torch.allclose(out.double(), ref, atol=2e-5), f"chunk {step}"
    assert differed, "the stream never made two heads keep different tokens: the per-head positions were not exercised"


def test_chunked_with_cache_equals_dense_single_shot():
    """cascade/models/test.py:123-165: while the whole stream fits (C == 1), chunked attention
    through the cache equals ordinary causal attention with ordinary positions."""
    g = torch.Generator().manual_seed(2)
    B, H, KVH, D, NS, W = 1, 4, 4, 16, 4, 64
    n, stride = 60, 7
    q, k, v = rand_chunk(g, B, H, KVH, n, D)
    pos = torch.arange(n)
    ref = F.scaled_dot_product_attention(rope_complex(q, pos, 5e5), rope_complex(k, pos, 5e5), v.double(),
                                         is_causal=True)
    cache, attn = make_layer(B, H, KVH, D, NS, W, 1, eager=True, theta=5e5)
    outs = []
    first = q[:, :, :stride]  # later chunks may not be longer than the first (cascade_attention.py:120-123)
    assert first.size(2) == stride
    for i in range(0, n, stride):
        outs.append(attn.forward(q[:, :, i:i + stride], k[:, :, i:i + stride], v[:, :, i:i + stride], cache))
    out = torch.cat(outs, dim=2)
    assert torch.allclose(out.double(), ref, atol=2e-5)


@pytest.mark.parametrize("reduction", ["mean", "max", "median"])
@pytest.mark.parametrize("homogeneous", [False, True])
def test_score_sums_closed_form(reduction, homogeneous):
    g = torch.Generator().manual_seed(3)
    B, H, KVH, D, NS, W, C, Q = 1, 6, 2, 8, 2, 4, 2, 5
    cache, attn = make_layer(B, H, KVH, D, NS, W, C, True, reduction=reduction, homogeneous=homogeneous)
    cache.beta = 0.9  # make the geometric weights visible in fp32
    for step in range(4):
        q, k, v = rand_chunk(g, B, H, KVH, Q, D)
        vals = cache.get_vals()
        q_pos = torch.arange(Q) + (0 if step == 0 else max(int(vals[2].max()), int(vals[6].max())) + 1)
        _, p, n_prev = dense_reference(q, k, v, cache, 10000.0, q_pos)
        valid = ~cache.mask[0, 0]
        n_sink_valid = int((~cache.sink_mask[0, 0]).sum())
        before = cache.score_cache.clone().double()
        og_before = cache.og_pos.clone()
        attn.forward(q, k, v, cache)
        beta = 0.9
        # float64 loops straight from the definitions (cascade_attention.py:270-282, 315-323)
        ema = torch.zeros(B, H, W * C, dtype=torch.float64)
        cols = torch.nonzero(valid).flatten().tolist()
        for j, slot in enumerate(cols):
            for m in range(Q):
                ema[:, :, slot] += (1 - beta) * beta ** (Q - 1 - m) * p[:, :, m, n_sink_valid + j]
        new = torch.zeros(B, H, Q, dtype=torch.float64)
        for n_ in range(Q):
            for m in range(n_, Q):
                new[:, :, n_] += (1 - beta) * beta ** (m - n_) * p[:, :, m, n_prev + n_]
        red = {"mean": lambda x: x.mean(2), "max": lambda x: x.amax(2),
               "median": lambda x: x.median(2).values}[reduction]
        if homogeneous:
            ema_r = red(ema.view(B, 1, H, -1)).expand(B, KVH, -1)
            new_r = red(new.view(B, 1, H, -1)).expand(B, KVH, -1)
        else:
            ema_r = red(ema.view(B, KVH, H // KVH, -1))
            new_r = red(new.view(B, KVH, H // KVH, -1))
        # the EMA tail happens before the update scatters, so compare what went INTO the update
        assert torch.allclose(attn.last_ema.double().expand(B, KVH, -1), ema_r, atol=1e-6)
        assert torch.allclose(attn.last_new_scores[:, :KVH].double(), new_r, atol=1e-6)
        expect_cache = beta ** Q * before + ema_r
        # slots whose token stayed put through the update hold the decayed EMA plus the increment
        stayed = (og_before == cache.og_pos) & valid[None, None, :]
        assert torch.allclose(cache.score_cache.double()[stayed], expect_cache[stayed], atol=1e-6)


def test_decode_step_closed_form():
    """q == 1: ema = (1-beta) * P[0, slot], new score = (1-beta) * P[0, last]."""
    g = torch.Generator().manual_seed(4)
    B, H, KVH, D, NS, W, C = 2, 4, 2, 8, 2, 4, 2
    cache, attn = make_layer(B, H, KVH, D, NS, W, C, True)
    q, k, v = rand_chunk(g, B, H, KVH, 7, D)
    attn.forward(q, k, v, cache)
    q, k, v = rand_chunk(g, B, H, KVH, 1, D)
    vals = cache.get_vals()
    q_pos = torch.arange(1) + max(int(vals[2].max()), int(vals[6].max())) + 1
    ref, p, n_prev = dense_reference(q, k, v, cache, 10000.0, q_pos)
    before = cache.score_cache.clone()
    nvalid = int((~vals[7][0, 0]).sum())  # counted before the update fills another slot
    out = attn.forward(q, k, v, cache)
    assert torch.allclose(out.double(), ref, atol=2e-5)
    beta = cache.beta
    new = (1 - beta) * p[:, :, 0, -1].view(B, KVH, H // KVH).mean(-1)
    assert torch.allclose(attn.last_new_scores[:, :KVH, 0].double(), new, rtol=1e-4, atol=1e-12)
    ema = (1 - beta) * p[:, :, 0, NS:NS + nvalid].view(B, KVH, H // KVH, -1).mean(2)
    assert torch.allclose(attn.last_ema[:, :, :nvalid].double(), ema, rtol=1e-4, atol=1e-12)
    assert before.shape == cache.score_cache.shape


def test_head_reduction_groups_follow_repeat_kv_order():
    """kv head g serves query heads g*G .. g*G+G-1 (modeling_llama.py:316-325)."""
    B, H, KVH, S, Q = 1, 6, 2, 3, 2
    scores = torch.arange(H, dtype=torch.float32).view(1, H, 1).expand(B, H, S + Q).contiguous()
    ema, new = calc_scores(scores, False, S, Q, KVH, "mean")
    assert ema[0, :, 0].tolist() == [1.0, 4.0] and new[0, :, 0].tolist() == [1.0, 4.0]
    ema, new = calc_scores(scores, False, S, Q, KVH, "max")
    assert ema[0, :, 0].tolist() == [2.0, 5.0]
    ema, new = calc_scores(scores, False, S, Q, KVH, "median")
    assert ema[0, :, 0].tolist() == [1.0, 4.0]
    ema, new = calc_scores(scores, True, S, Q, KVH, "median")  # lower median of 0..5
    assert ema.shape == (1, 1, S) and ema[0, 0, 0].item() == 2.0 and new.shape == (1, KVH, Q)
