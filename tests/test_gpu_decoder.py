"""The generation loop of the reference (cascade_attention.py:452-538: prompt in strides, then one token at
a time) over a small multi-layer decoder: every layer owns one layer of a CascadingKVCache.  The CPU side
is the same decoder with the oracle's attention and one OracleCache per layer."""
import pytest
import torch

from oracle.attention import OracleCascadeAttention
from oracle.update import OracleCache

from parity_helpers import (META, FlipLedger, assert_scores_close, check_update_against_replay, clone_oracle,
                            flip_bound, flip_margins, push_state, tol)

pytestmark = pytest.mark.gpu


def oracle_logits(model, oracles, caches, ids):
    cfg = model.cfg
    B, q = ids.shape
    x = model.embed_tokens(ids)
    for layer, attn_o, cache in zip(model.layers, oracles, caches):
        h = layer.input_layernorm(x)
        qs, ks, vs = layer.self_attn.qkv(h, (B, q, cfg.num_heads, cfg.head_dim), (B, q, cfg.num_kv_heads, cfg.head_dim))
        a = attn_o.forward(qs, ks, vs, cache)
        x = x + layer.self_attn.o_proj(a.transpose(1, 2).reshape(B, q, -1))
        x = x + layer.mlp(layer.post_attention_layernorm(x))
    return model.lm_head(model.norm(x[:, -1:]))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_decoder_prefill_and_greedy_steps_against_the_oracle(dtype):
    from cascading_kv_cache_amd.decoder import PRESETS, CascadeDecoder

    cfg = PRESETS["tiny"]
    gpu = CascadeDecoder(cfg, dtype=dtype, device="cuda:0", seed=3)
    cpu = CascadeDecoder(cfg, dtype=dtype, device="cpu", seed=3)
    for (n1, p1), (n2, p2) in zip(gpu.named_parameters(), cpu.named_parameters()):
        assert n1 == n2 and torch.equal(p1.cpu(), p2), n1
    B, NS, W, C = 2, 4, 64, 2      # the stream below stays inside the window: no eviction, so no score ties decide
    cache = gpu.new_cache(W * C, C, batch=B, num_sink_tokens=NS)
    caches = [OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=cfg.num_kv_heads,
                          dim=cfg.head_dim, max_seq_len=W * C, dtype=dtype) for _ in range(cfg.num_layers)]
    oracles = [OracleCascadeAttention(cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, rope_theta=cfg.rope_theta,
                                      head_reduction=cfg.head_reduction) for _ in range(cfg.num_layers)]
    ids = torch.randint(0, cfg.vocab_size, (B, 70), generator=torch.Generator().manual_seed(4))
    with torch.no_grad():
        steps = [ids[:, 0:32], ids[:, 32:64], ids[:, 64:70]] + [ids[:, i:i + 1] for i in range(5)]
        for n, chunk in enumerate(steps):
            lg = gpu(chunk.cuda(), cache).float().cpu()
            lc = oracle_logits(cpu, oracles, caches, chunk).float()
            scale = lc.abs().max().item()
            err = (lg - lc).abs().max().item()
            assert err <= 3e-2 * scale + 1e-3, f"step {n}: logits differ by {err:.3e} (scale {scale:.3e})"
    seen = cache.seen_tokens_by_layer.cpu().tolist()
    assert seen == [75] * cfg.num_layers, seen
    for i, oc in enumerate(caches):
        for name in ("mask", "sink_mask", "pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks", "og_pos"):
            assert torch.equal(getattr(cache, name)[i].cpu(), getattr(oc, name)), f"layer {i}: {name}"


@pytest.mark.parametrize("dtype,layer_sizes", [(torch.bfloat16, None), (torch.float16, None),
                                               (torch.bfloat16, [(32, 4), (16, 2)]), (torch.float16, [(8, 8), (64, 1)])])
def test_decoder_layers_past_the_window_teacher_forced(dtype, layer_sizes):
    """``layer_sizes``: (slots per ring, rings) of every layer when the layers differ in size, as the caches of
    cascade/models/test.py:325-377 do (per-layer ``window_length`` / ``max_seq_len`` lists).

    The multi-layer path once the cascades evict: a stream of more than twice the window goes through a
    two-layer decoder in strides and then token by token.  Every layer's cache layer restarts each step from
    that layer's oracle state and the oracle's attention gets the device's own q/k/v, so a tie-level decision
    cannot snowball; per layer and step the attention output, both score inputs, the metadata, the update
    (against the oracle's update on the library's scores) and the margin of every differing slot are checked."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq
    from cascading_kv_cache_amd.decoder import PRESETS, CascadeDecoder

    cfg = PRESETS["tiny"]
    model = CascadeDecoder(cfg, dtype=dtype, device="cuda:0", seed=7)
    B, NS = 2, 4
    sizes = layer_sizes or [(32, 4)] * cfg.num_layers
    if layer_sizes:
        cache = model.new_cache([w * c for w, c in sizes], [c for _, c in sizes], batch=B, num_sink_tokens=NS)
        assert cache.window_length == [w for w, _ in sizes] and cache.cascades == [c for _, c in sizes]
        assert [t.size(2) for t in cache.key_cache] == [w * c for w, c in sizes]
    else:
        cache = model.new_cache(32 * 4, 4, batch=B, num_sink_tokens=NS)
    caches = [OracleCache(window_length=w, num_sink_tokens=NS, max_batch_size=B, heads=cfg.num_kv_heads,
                          dim=cfg.head_dim, max_seq_len=w * c, dtype=dtype) for w, c in sizes]
    oracles = [OracleCascadeAttention(cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, rope_theta=cfg.rope_theta,
                                      head_reduction=cfg.head_reduction) for _ in range(cfg.num_layers)]
    inv_freq = default_inv_freq(cfg.head_dim, cfg.rope_theta, "cuda:0")
    steps = [48] * 6 + [1] * 14          # 302 tokens through caches of 4 sinks + at most 128 slots
    ids = torch.randint(0, cfg.vocab_size, (B, sum(steps)), generator=torch.Generator().manual_seed(8)).cuda()
    ledger = FlipLedger(dtype)
    done = 0
    with torch.no_grad():
        for n, qn in enumerate(steps):
            x = model.embed_tokens(ids[:, done:done + qn])
            for li, layer in enumerate(model.layers):
                oc, attn_o = caches[li], oracles[li]
                h = layer.input_layernorm(x)
                qs, ks, vs = layer.self_attn.qkv(h, (B, qn, cfg.num_heads, cfg.head_dim),
                                                 (B, qn, cfg.num_kv_heads, cfg.head_dim))
                push_state(cache, oc, layer=li)
                replay = clone_oracle(oc)
                pre = {"og_pos": oc.og_pos.clone(), "mask": oc.mask.clone()}
                seen_before = int(oc.seen_tokens)
                out_g, new_g = cascade_attention(qs, ks, vs, cache, li, inv_freq, head_reduction=cfg.head_reduction,
                                                 update_cache=False)
                scores_g = cache.score_cache[li].cpu().clone()
                cache.update(ks, vs, li, score_states=new_g)
                qc, kc, vc = qs.cpu(), ks.cpu(), vs.cpu()
                out_c = attn_o.forward(qc, kc, vc, oc)
                ctx = f"step {n} (q={qn}) layer {li}"
                err = (out_g.float().cpu() - out_c.float()).abs().max().item()
                assert err <= tol(dtype), f"{ctx}: out max err {err:.3e}"
                new_c = attn_o.last_new_scores[:, :cfg.num_kv_heads]
                eps = assert_scores_close(new_g, new_c, dtype, f"{ctx} new-token scores")
                eps = max(eps, assert_scores_close(scores_g, attn_o.last_score_cache, dtype, f"{ctx} score cache"))
                for name in META:
                    assert torch.equal(getattr(cache, name)[li].cpu(), getattr(oc, name)), f"{ctx}: {name}"
                check_update_against_replay(cache, replay, kc, vc, scores_g, new_g.cpu(), layer=li, ctx=ctx)
                og_g = cache.og_pos[li].cpu()
                margins = flip_margins(og_g, oc, pre, seen_before, attn_o.last_score_cache, new_c)
                ledger.record(margins, eps, og_g.numel(), primary_only=qn < 2 * sizes[li][0], ctx=ctx)
                x = x + layer.self_attn.o_proj(out_g.transpose(1, 2).reshape(B, qn, -1))
                x = x + layer.mlp(layer.post_attention_layernorm(x))
            done += qn
    print(ledger.summary())
    assert cache.seen_tokens_by_layer.cpu().tolist() == [done] * cfg.num_layers
    for oc in caches:
        assert not bool(oc.mask.any()) and int(oc.start_indices.sum()) > 0, "the cascades must have evicted"
    assert ledger.flips <= flip_bound(ledger), ledger.summary()


def test_generate_streams_past_the_window():
    from cascading_kv_cache_amd.decoder import PRESETS, CascadeDecoder, generate

    cfg = PRESETS["tiny"]
    model = CascadeDecoder(cfg, dtype=torch.bfloat16, device="cuda:0", seed=5)
    cache = model.new_cache(128, 4, batch=2, num_sink_tokens=4)
    ids = torch.randint(0, cfg.vocab_size, (2, 500), generator=torch.Generator().manual_seed(6)).cuda()
    out = generate(model, ids, cache, stride=96, max_new_tokens=12)
    assert out.shape == (2, 512) and torch.equal(out[:, :500], ids)
    assert int(out.min()) >= 0 and int(out.max()) < cfg.vocab_size
    # 500 prompt tokens + 11 fed-back tokens went through every layer (the last new token is never fed back)
    assert cache.seen_tokens_by_layer.cpu().tolist() == [511] * cfg.num_layers
    assert not bool(cache.mask[0].any()) and not bool(cache.mask[cfg.num_layers - 1].any())  # every slot holds a token


@pytest.mark.parametrize("preset_bias", [False, True])
def test_fused_projections_keep_the_decoder(preset_bias):
    """q/k/v and gate/up projections as one product each (weights as views of shared buffers) and one-kernel norms:
    the same decoder, prefill and single-token steps, up to the rounding of the norm."""
    from dataclasses import replace

    from cascading_kv_cache_amd.decoder import PRESETS, CascadeDecoder

    cfg = replace(PRESETS["tiny"], qkv_bias=preset_bias)
    dtype = torch.bfloat16
    plain = CascadeDecoder(cfg, dtype=dtype, device="cuda:0", seed=5)
    fused = CascadeDecoder(cfg, dtype=dtype, device="cuda:0", seed=5).fuse_projections()
    for (n1, p1), (n2, p2) in zip(plain.named_parameters(), fused.named_parameters()):
        assert n1 == n2 and torch.equal(p1, p2), n1
    B, NS, W, C = 2, 4, 32, 2
    ca, cb = (m.new_cache(W * C, C, batch=B, num_sink_tokens=NS) for m in (plain, fused))
    ids = torch.randint(0, cfg.vocab_size, (B, 100), generator=torch.Generator().manual_seed(6)).cuda()
    with torch.no_grad():
        for chunk in [ids[:, 0:40], ids[:, 40:80]] + [ids[:, 80 + i:81 + i] for i in range(20)]:
            la, lb = plain(chunk, ca).float(), fused(chunk, cb).float()
            scale = la.abs().max().item()
            assert (la - lb).abs().max().item() <= 2e-2 * scale + 1e-3
    for name in ("mask", "sink_mask", "pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks"):
        for i in range(cfg.num_layers):
            assert torch.equal(getattr(ca, name)[i], getattr(cb, name)[i]), f"layer {i}: {name}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_chunked_prefill_equals_one_dense_shot_while_the_stream_fits(dtype):
    """cascade/models/test.py:123-165 on the device: sinks 64, window 2048 as one cascade, stride 128, a 988-token
    prompt.  While nothing has been evicted, streaming the prompt through the cache in strides gives the logits of
    one dense causal pass over the whole prompt (here: the same decoder fed the prompt as a single chunk into a fresh
    cache, which is plain causal attention with ordinary positions): within 1e-1 of each other relative to the
    logits' scale, and the same argmax wherever the dense pass's best logit leads by more than that tolerance."""
    from cascading_kv_cache_amd.decoder import PRESETS, CascadeDecoder

    cfg = PRESETS["tiny"]
    model = CascadeDecoder(cfg, dtype=dtype, device="cuda:0", seed=11)
    n, stride = 988, 128
    ids = torch.randint(0, cfg.vocab_size, (1, n), generator=torch.Generator().manual_seed(12)).cuda()
    with torch.no_grad():
        dense = model(ids, model.new_cache(2048, 1, batch=1, num_sink_tokens=64), last_only=False).float()
        cache = model.new_cache(2048, 1, batch=1, num_sink_tokens=64)
        chunked = torch.cat([model(ids[:, i:i + stride], cache, last_only=False) for i in range(0, n, stride)], 1).float()
    assert chunked.shape == dense.shape == (1, n, cfg.vocab_size)
    scale = dense.abs().max().item()
    err = (chunked - dense).abs().max().item()
    rel = 1e-4 if dtype == torch.float32 else 3e-2
    assert err <= rel * scale, f"{dtype}: logits differ by {err:.3e} (scale {scale:.3e})"
    top2 = dense.topk(2, dim=-1).values
    clear = (top2[..., 0] - top2[..., 1]) > 2 * rel * scale
    # float32 leaves nearly every position with a clear winner; at the 16-bit tolerance about four in ten
    assert int(clear.sum()) > (n // 2 if dtype == torch.float32 else n // 4), "too few clear winners to compare"
    assert torch.equal(chunked.argmax(-1)[clear], dense.argmax(-1)[clear])
    assert cache.seen_tokens_by_layer.cpu().tolist() == [n] * cfg.num_layers
    assert int(cache.start_indices[0].sum()) == 0, "nothing may have been evicted"
