"""Pins the CPU update oracle (oracle/ckv_oracle_update.c) before anything is compared to it.

Each test checks the oracle against something that does not share its code: closed forms,
special cases with textbook answers, invariants of the data structure, an independent
restatement of the reference's per-token ``CascadingKVCacheSlow`` and the procedural checks of
the reference's own test file (cascade/models/test.py:325-377, 423-497, 499-651).
"""
import random

import pytest
import torch

from oracle.update import CASCADE_FUNCS, OracleCache, acceptance_periods

from slow_cache_restated import SlowCacheRestated


def token_stream(n, heads=1, dim=1, batch=1, dtype=torch.float32, start=0):
    """keys whose every element equals the 1-based token index (as in test.py:412-415)."""
    k = (torch.arange(n, dtype=torch.float32) + start + 1).to(dtype)
    return k.view(1, 1, -1, 1).repeat(batch, heads, 1, dim).contiguous()


def feed(cache, k, chunk, scores=None):
    n = k.size(2)
    for i in range(0, n, chunk):
        s = None if scores is None else scores[:, :, i:i + chunk].contiguous()
        cache.update(k[:, :, i:i + chunk].contiguous(), (k[:, :, i:i + chunk] * 2).contiguous(), s)


# ---------------------------------------------------------------------------------------------
def test_sink_phase_closed_form():
    NS = 5
    c = OracleCache(window_length=4, num_sink_tokens=NS, max_batch_size=2, heads=3, dim=2, max_seq_len=8)
    c.pos.fill_(-7)  # must stay untouched: no position pass while only sinks are written
    feed(c, token_stream(3, heads=3, dim=2, batch=2), 3)
    assert c.stored_sinks.eq(3).all()
    assert c.sink_keys[..., :3, 0].eq(torch.tensor([1.0, 2.0, 3.0])).all()
    assert c.sink_values[..., :3, 1].eq(torch.tensor([2.0, 4.0, 6.0])).all()
    assert c.sink_pos[..., :3].eq(torch.tensor([0, 1, 2])).all()
    assert (~c.sink_mask[..., :3]).all() and c.sink_mask[..., 3:].all()
    assert c.pos.eq(-7).all() and c.mask.all() and c.stored_tokens.eq(0).all()
    # a chunk that straddles the boundary: 2 more sinks, then 3 cache tokens
    feed(c, token_stream(5, heads=3, dim=2, batch=2, start=3), 5)
    assert c.stored_sinks.eq(NS).all() and (~c.sink_mask).all()
    assert c.key_cache[0, 0, :3, 0].tolist() == [6.0, 7.0, 8.0]
    assert c.og_pos[1, 2, :3].tolist() == [6, 7, 8]
    assert c.pos[0, 0, :4].tolist() == [0, 1, 2, 0]  # (j + seg) % seg + ub - seg with seg = ub = 3
    # get_vals adds the sink count once more tokens than sinks were seen (cascading_cache.py:1282-1292)
    assert c.get_vals()[6][0, :3].tolist() == [NS, NS + 1, NS + 2]


@pytest.mark.parametrize("eager_fill", [False, True])
@pytest.mark.parametrize("chunk", [1, 3, 64])
def test_single_cascade_is_streaming_llm(eager_fill, chunk):
    """C == 1: sinks are the first NSINK tokens, the ring holds the last W (StreamingLLM)."""
    NS, W, n = 4, 16, 150
    c = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=1, heads=2, dim=3, max_seq_len=W,
                    eager_fill=eager_fill)
    feed(c, token_stream(n, heads=2, dim=3), chunk)
    assert c.sink_keys[0, 0, :, 0].tolist() == [1.0, 2.0, 3.0, 4.0]
    last = list(range(n - W + 1, n + 1))  # 1-based ids of the W most recent tokens
    for tok in last:
        slot = (tok - 1 - NS) % W  # ring: u-th non-sink token lives in slot u mod W
        assert c.key_cache[0, 1, slot, 2].item() == float(tok)
        assert c.og_pos[0, 1, slot].item() == tok
        assert c.pos[0, 1, slot].item() == tok - last[0]
    assert c.start_indices[0, 0, 0].item() == (n - NS) % W
    assert not c.mask.any()


def check_invariants(c: OracleCache, zero_scores: bool):
    W, C = c.window_length, c.cascades
    for b in range(c.max_batch_size):
        for h in range(c.heads):
            st = c.stored_tokens[b, h].tolist()
            sx = c.start_indices[b, h].tolist()
            for i in range(C):
                assert 0 <= st[i] <= W and 0 <= sx[i] < W
                if st[i] < W:
                    assert sx[i] == 0
                if i + 1 < C and st[i + 1] > 0:
                    assert st[i] == W, "cascades fill strictly in order"
                m = c.mask[b, h, i * W:(i + 1) * W]
                assert (~m[:st[i]]).all() and m[st[i]:].all()
            if int(c.stored_sinks[b, h]) < c.num_sink_tokens:
                continue
            valid = ~c.mask[b, h]
            pos = c.pos[b, h][valid]
            total = sum(st)
            assert sorted(pos.tolist()) == list(range(total)), "compact positions are a permutation"
            og = c.og_pos[b, h][valid]
            order = torch.argsort(pos)
            og_sorted = og[order].tolist()
            if zero_scores:
                assert all(x < y for x, y in zip(og_sorted, og_sorted[1:])), "position order == age order"
            for i in range(C - 1):  # everything in a deeper cascade is older
                if st[i + 1] > 0:
                    a = c.og_pos[b, h, i * W:i * W + st[i]]
                    d = c.og_pos[b, h, (i + 1) * W:(i + 1) * W + st[i + 1]]
                    if zero_scores:
                        assert d.max() < a.min()
            # stored payload agrees with og_pos (keys carry their own token index)
            assert c.key_cache[b, h][valid][:, 0].long().tolist() == og.tolist()


@pytest.mark.parametrize("seed", range(6))
def test_metadata_invariants_and_score_independence(seed):
    rng = random.Random(seed)
    NS = rng.choice([0, 1, 4, 7])
    W = rng.choice([1, 2, 3, 4, 8])
    C = rng.choice([1, 2, 3, 4, 5])
    func = rng.choice(CASCADE_FUNCS)
    eager = rng.random() < 0.5
    n = rng.randint(1, 40 * W)
    kw = dict(window_length=W, num_sink_tokens=NS, max_batch_size=1, heads=2, dim=1, max_seq_len=W * C,
              cascade_func=func, eager_fill=eager)
    a, b = OracleCache(**kw), OracleCache(**kw)
    k = token_stream(n, heads=2)
    g = torch.Generator().manual_seed(seed)
    scores = torch.randint(0, 3, (1, 2, n), generator=g).float()
    done = 0
    while done < n:
        q = rng.randint(1, 2 * W + 3)
        ks = k[:, :, done:done + q].contiguous()
        a.update(ks, ks.clone())
        b.update(ks, ks.clone(), scores[:, :, done:done + q].contiguous())
        done += q
        check_invariants(a, zero_scores=True)
        check_invariants(b, zero_scores=False)
        for name in ("stored_tokens", "start_indices", "stored_sinks", "mask", "sink_mask", "pos", "sink_pos"):
            assert torch.equal(getattr(a, name), getattr(b, name)), f"{name} must not depend on scores"


def test_eager_fill_fills_everything():
    """cascade/models/test.py:325-377: with eager fill, S + NSINK (or more) tokens leave nothing masked."""
    rng = random.Random(0)
    for _ in range(8):
        S = rng.choice([32, 64, 128])
        C = rng.choice([1, 2, 4, 8])
        NS = 8
        n = rng.randint(S + NS, 2 * S)
        c = OracleCache(window_length=S // C, num_sink_tokens=NS, max_batch_size=1, heads=1, dim=4, max_seq_len=S)
        c.update(torch.randn(1, 1, n, 4), torch.randn(1, 1, n, 4))
        assert c.mask.sum().item() == 0 and c.key_cache.size(2) == S
    # exactly S + NSINK tokens: the last one (0-based index S+NSINK-1) is still accepted everywhere
    c = OracleCache(window_length=4, num_sink_tokens=2, max_batch_size=1, heads=1, dim=1, max_seq_len=16)
    feed(c, token_stream(18), 18)
    assert c.mask.sum().item() == 0
    assert sorted(c.og_pos.view(-1).tolist()) == list(range(3, 19))
    # and the token with 0-based index S+NSINK as well (`<=`, cascading_cache.py:440, 471)
    feed(c, token_stream(1, start=18), 1)
    assert sorted(c.og_pos.view(-1).tolist()) == list(range(4, 20))


@pytest.mark.parametrize("seed", range(8))
def test_eager_fill_query_positions_follow_the_token_counter(seed):
    """With eager fill nothing is dropped before the cache is full, so the id the next chunk starts at (one past the
    largest id among sinks and slots, stale entries included, cascade_attention.py:119-150) is min(seen, S + NSINK):
    what the host side hands out without reading the device."""
    rng = random.Random(100 + seed)
    NS = rng.choice([0, 1, 4, 7])
    W = rng.choice([1, 2, 3, 4, 8])
    C = rng.choice([1, 2, 3, 4, 5])
    func = rng.choice(CASCADE_FUNCS)
    c = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=1, heads=2, dim=1, max_seq_len=W * C,
                    cascade_func=func, eager_fill=True)
    n = rng.randint(1, 6 * W * C + NS)
    k = token_stream(n, heads=2)
    g = torch.Generator().manual_seed(seed)
    scores = torch.rand(1, 2, n, generator=g)
    done = 0
    while done < n:
        q = rng.randint(1, 2 * W + 3)
        c.update(k[:, :, done:done + q].contiguous(), k[:, :, done:done + q].clone(), scores[:, :, done:done + q].contiguous())
        done = min(done + q, n)
        seen = int(c.seen_tokens)
        shift = NS if seen > NS else 0
        largest = int(c.pos[0, 0].amax()) + shift
        if NS:
            largest = max(largest, int(c.sink_pos[0, 0].amax()))
        assert largest + 1 == min(seen, W * C + NS), (seen, largest)


def test_eager_add_same_as_one_cascade():
    """cascade/models/test.py:423-497."""
    for S in (32, 64, 128):
        NS = 8
        sllm = OracleCache(window_length=S, num_sink_tokens=NS, max_batch_size=1, heads=1, dim=1, max_seq_len=S,
                           eager_fill=False)
        ours = OracleCache(window_length=S // 4, num_sink_tokens=NS, max_batch_size=1, heads=1, dim=1,
                           max_seq_len=S, eager_fill=True)
        k = token_stream(S)
        feed(sllm, k, 1)
        feed(ours, k, S)
        for x, y in zip(sllm.get_vals(), ours.get_vals()):
            have = set(x.reshape(-1).tolist())
            assert all(v in have for v in y.reshape(-1).tolist())


@pytest.mark.parametrize("seed", range(5))
def test_split_call_invariance(seed):
    rng = random.Random(100 + seed)
    NS, W, C = rng.choice([0, 3, 4]), rng.choice([2, 4, 8]), rng.choice([2, 3, 4])
    eager = bool(seed % 2)
    n = rng.randint(NS + 1, 30 * W)
    kw = dict(window_length=W, num_sink_tokens=NS, max_batch_size=2, heads=2, dim=2, max_seq_len=W * C,
              dtype=torch.bfloat16, eager_fill=eager)
    whole, single, ragged = OracleCache(**kw), OracleCache(**kw), OracleCache(**kw)
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(2, 2, n, 2, generator=g).to(torch.bfloat16)
    s = (torch.randint(0, 4, (2, 2, n), generator=g).float() / 8).to(torch.bfloat16)
    feed(whole, k, n, s)
    feed(single, k, 1, s)
    done = 0
    while done < n:
        q = rng.randint(1, 3 * W)
        ragged.update(k[:, :, done:done + q].contiguous(), (k[:, :, done:done + q] * 2).contiguous(),
                      s[:, :, done:done + q].contiguous())
        done += q
    for name, t in whole.state_dict().items():
        assert torch.equal(t, single.state_dict()[name]), name
        assert torch.equal(t, ragged.state_dict()[name]), name


@pytest.mark.parametrize("W,S,NS", [(4, 32, 64), (4, 32, 3), (8, 32, 0), (2, 16, 5), (16, 64, 4)])
def test_against_restated_slow_cache_every_token(W, S, NS):
    """cascade/models/test.py:499-651: after EVERY token, keys sorted by position id and the
    position ids themselves agree with the reference's independent per-token implementation."""
    n = 300 + NS
    slow = SlowCacheRestated(W, NS, S)
    fast = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=1, heads=2, dim=1, max_seq_len=S,
                       eager_fill=False)
    k = token_stream(n, heads=2)
    for t in range(n):
        pos_slow = slow.update(float(t + 1))
        _, _, _, _, kc, _, pos_fast, mask, _ = fast.update(k[:, :, t:t + 1].contiguous(), k[:, :, t:t + 1].contiguous())
        nvalid = int((~mask[0, 0]).sum())
        assert nvalid == sum(not m for m in slow.masked)
        assert pos_fast[0, :nvalid].tolist() == pos_slow[:nvalid]
        order_f = torch.argsort(pos_fast[0, :nvalid])
        keys_f = kc[0, 1, :nvalid, 0][order_f].tolist()
        order_s = sorted(range(nvalid), key=lambda j: pos_slow[j])
        assert keys_f == [slow.keys[j] for j in order_s]
        assert fast.sink_keys[0, 0, :len(slow.sinks), 0].tolist() == slow.sinks


def test_against_restated_slow_cache_batched():
    """cascade/models/test.py:653-807: one batched call equals the per-token implementation."""
    rng = random.Random(3)
    W, S, NS = 16, 64, 8
    for _ in range(3):
        n = rng.randint(200, 1500)
        slow = SlowCacheRestated(W, NS, S)
        for t in range(n):
            pos_slow = slow.update(float(t + 1))
        fast = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=1, heads=1, dim=1, max_seq_len=S,
                           eager_fill=False)
        k = token_stream(n)
        _, _, _, _, kc, _, pos_fast, mask, _ = fast.update(k, k.clone())
        nvalid = int((~mask[0, 0]).sum())
        order_f = torch.argsort(pos_fast[0, :nvalid])
        order_s = sorted(range(nvalid), key=lambda j: pos_slow[j])
        assert kc[0, 0, :nvalid, 0][order_f].tolist() == [slow.keys[j] for j in order_s]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_tournament_is_last_group_maximum(dtype):
    """Two cascades, the second never fills: its content has a closed form.

    Cascade 0 is a FIFO of W slots, so non-sink token u is evicted when token u+W arrives, at
    global 0-based index g = NS+u+W.  Cascade 1 appends it when (g-NS) % 2 == 0, otherwise it
    competes with the newest slot and wins iff score >= (cascading_cache.py:699).  Each slot of
    cascade 1 therefore ends up holding the LAST maximum of its group of consecutive arrivals.
    """
    NS, W, W1 = 2, 4, 64
    # C=2 needs equal windows, so emulate "never fills" with a large common window and few tokens
    W = W1
    n_tokens = NS + W + 60
    g = torch.Generator().manual_seed(7)
    scores = (torch.randint(0, 5, (1, 1, n_tokens), generator=g).float() / 4).to(dtype)  # tie-heavy
    c = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=1, heads=1, dim=1, max_seq_len=2 * W,
                    dtype=dtype, eager_fill=False)
    k = token_stream(n_tokens, dtype=dtype)
    feed(c, k, 7, scores)
    expected = []  # list of (token id, score)
    for u in range(0, n_tokens - NS - W):  # evicted non-sink tokens, in order
        tok, sc = NS + u + 1, scores[0, 0, NS + u].item()
        if (u + W) % 2 == 0 or not expected:
            expected.append((tok, sc))
        elif sc >= expected[-1][1]:
            expected[-1] = (tok, sc)
    got = list(zip(c.og_pos[0, 0, W:W + len(expected)].tolist(), c.score_cache[0, 0, W:W + len(expected)].tolist()))
    assert got == expected
    assert c.stored_tokens[0, 0].tolist() == [W, len(expected)]


def test_acceptance_period_tables():
    assert acceptance_periods("pow2", 4) == [1, 2, 4, 8]
    assert acceptance_periods("pow2-1", 4) == [1, 1, 1, 8]
    assert acceptance_periods("pow2-1-4", 8) == [1, 1, 1, 1, 1, 1, 64, 128]
    assert acceptance_periods("pow2-2-4", 8) == [1, 1, 1, 1, 16, 32, 64, 128]
    assert acceptance_periods("pow2-3-4", 8) == [1, 1, 4, 8, 16, 32, 64, 128]
    assert acceptance_periods("1-then-2", 4) == [1, 2, 2, 2]
    assert acceptance_periods("pow3", 3) == [1, 3, 9]
    assert acceptance_periods("pow4", 3) == [1, 4, 16]
    assert acceptance_periods("iplus1", 4) == [1, 2, 3, 4]
    with pytest.raises(ValueError):
        acceptance_periods("nope", 4)
