"""Shared pieces of the GPU parity tests: teacher forcing, bit-level comparison, and the analysis of
eviction decisions that differ between the library and the oracle.

Why decisions may differ at all.  The update is bit-exact given identical scores (tests/test_gpu_update.py),
but its score inputs come from the attention kernels, which agree with the oracle to a tolerance, not to
the bit.  The tournament "the later arrival stays iff its score >= the kept one's"
(cascade/models/cascading_cache.py:699) keeps the last arrival with the largest score, so two score sets that
differ by at most eps per element can only disagree between tokens whose oracle scores lie within 2 eps of
each other.  ``check_update_against_replay`` proves the first half (the oracle's update fed with the
library's scores reproduces the library's state bit for bit); ``flip_margins`` measures the second.
"""
import copy

import torch

STATE = ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask", "pos",
         "og_pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")
META = ("mask", "sink_mask", "pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")
ULP = {torch.float32: 2.0 ** -23, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -10}


def tol(dtype):
    """Absolute tolerance of attention outputs stated for this path: 1e-4 in float32, 2e-2 in 16-bit."""
    return 1e-4 if dtype == torch.float32 else 2e-2


def bits(t):
    """Floating tensors as integers, so that NaN payloads and signed zeros count in comparisons."""
    if t.dtype.is_floating_point:
        return t.view(torch.int16 if t.element_size() == 2 else torch.int32)
    return t


def push_state(gpu, cpu, layer=0):
    """Teacher forcing: layer ``layer`` of the GPU cache restarts from the oracle's state."""
    for name in STATE:
        getattr(gpu, name)[layer].copy_(getattr(cpu, name))
    gpu.seen_tokens_by_layer[layer] = int(cpu.seen_tokens)
    gpu._seen_host[layer] = int(cpu.seen_tokens)


def assert_scores_close(got, want, dtype, what):
    """Scores are 1e-7-scale numbers: compared relative to their largest magnitude with the tolerance of
    the outputs, plus one unit in the last place of the storage format."""
    got, want = got.float().cpu(), want.float().cpu()
    scale = want.abs().max().item() + 1e-30
    # float16 scores live among the subnormals (1e-7 ~ 2 * 2^-24): allow two quanta of the format
    quantum = 2.0 ** -24 if dtype == torch.float16 else 0.0
    err = (got - want).abs().max().item()
    assert err <= (tol(dtype) + ULP[dtype]) * scale + 2 * quantum, f"{what}: max err {err:.3e} vs scale {scale:.3e}"
    return err


def check_update_against_replay(gpu, replay, k, v, scores_after_attention, new_scores, layer=0, ctx=""):
    """``replay``: a copy of the oracle cache as it was BEFORE the chunk.  It is given the library's own score
    inputs (the score cache after the attention call, the chunk's new scores) and updated by the oracle; every
    state tensor of the GPU cache must then equal it bit for bit: with the same scores the library takes
    exactly the decisions of the serial reference loop."""
    replay.score_cache = scores_after_attention.clone()
    replay.update(k, v, new_scores)
    for name in STATE:
        g, w = bits(getattr(gpu, name)[layer].cpu()), bits(getattr(replay, name))
        if not torch.equal(g, w):
            bad = (g != w).nonzero()[:4].tolist()
            raise AssertionError(f"{ctx}: {name} differs from the oracle's update run on the library's scores, at {bad}")


def flip_margins(gpu_og, cpu, pre, seen_before, oracle_scores_after_attention, oracle_new_scores):
    """Slots whose token differs between the library and the oracle after an update, each with the distance
    between the ORACLE's scores of the two tokens that competed for it (the decision margin).

    gpu_og ``(B, KVH, S)`` int64 on the CPU; ``pre``: the oracle's og_pos and mask before the chunk;
    oracle_scores_after_attention ``(B, KVH, S)``: what evicted tokens carry; oracle_new_scores ``(B, >=KVH, q)``.
    Returns ``[(b, h, slot, token_gpu, token_cpu, margin), ...]``."""
    out = []
    diff = (gpu_og != cpu.og_pos).nonzero().tolist()
    for b, h, slot in diff:
        pair = []
        for token in (int(gpu_og[b, h, slot]), int(cpu.og_pos[b, h, slot])):
            if token > seen_before:  # a token of this chunk
                pair.append(float(oracle_new_scores[b, h, token - seen_before - 1]))
            else:                    # it sat in the cache before the chunk
                where = ((pre["og_pos"][b, h] == token) & ~pre["mask"][b, h]).nonzero()
                assert where.numel() == 1, f"token {token} not found among the cached tokens of ({b}, {h})"
                pair.append(float(oracle_scores_after_attention[b, h, int(where[0, 0])]))
        out.append((b, h, slot, int(gpu_og[b, h, slot]), int(cpu.og_pos[b, h, slot]), abs(pair[0] - pair[1])))
    return out


class FlipLedger:
    """Accumulates, over the chunks of a stream, how many slots chose a different token and how wide the
    oracle's margin was where they did."""

    def __init__(self, dtype):
        self.dtype = dtype
        self.flips = 0
        self.compared = 0
        self.decisions = 0           # slots rewritten by tournaments or inserts: where a decision could flip
        self.worst_ratio = 0.0       # largest margin / (2 eps) seen on a flip that is checked
        self.min_margin = float("inf")
        self.max_margin = 0.0

    def record(self, margins, eps, n_slots, primary_only, ctx):
        self.flips += len(margins)
        self.compared += n_slots
        for b, h, slot, tg, tc, m in margins:
            self.min_margin = min(self.min_margin, m)
            self.max_margin = max(self.max_margin, m)
            if primary_only:
                # the two tokens met in one tournament: their oracle scores cannot be further apart than twice
                # the largest difference between the two score sets
                assert m <= 2 * eps * (1 + 1e-6) + 1e-45, (
                    f"{ctx}: slot ({b}, {h}, {slot}) keeps token {tg} where the oracle keeps {tc}, but the oracle's "
                    f"scores of the two differ by {m:.3e} > 2 x {eps:.3e} (largest score difference)")
                if eps > 0:
                    self.worst_ratio = max(self.worst_ratio, m / (2 * eps))

    def summary(self):
        if not self.flips:
            return f"{self.dtype}: 0/{self.compared} slots differ"
        return (f"{self.dtype}: {self.flips}/{self.compared} slots chose a different token; oracle margin on those "
                f"slots {self.min_margin:.3e} .. {self.max_margin:.3e} (worst {self.worst_ratio:.2f} of the 2-eps bound)")


def flip_bound(ledger):
    """How many slots of a 16-bit stream may hold another token than the oracle's (each of them already shown to be a
    tie at the score tolerance): 0.25 % of the slots compared over the stream, about twice the largest rate measured
    on any test stream (18 of 16384 slots; the streams of a few thousand slots show 0 to 2), and never fewer than 3
    so that the smallest streams are not held to a fraction of a slot."""
    return max(3, int(0.0025 * ledger.compared))


def clone_oracle(cpu):
    return copy.deepcopy(cpu)
