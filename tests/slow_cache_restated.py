"""Independent cross-check for the update oracle: a scalar restatement of the reference's
per-token PyTorch cache ``CascadingKVCacheSlow`` and its helpers
(cascade/models/cascading_cache.py:1351-1494, 1496-1843).

It is a DIFFERENT algorithm from the kernel the oracle restates: one token per call, position ids
maintained incrementally per visited cascade (update_segment_pos, :1351-1366) instead of being
recomputed for the whole cache, acceptance flags derived from a counter that is incremented
before the insertion (set_cache_bools, :1680-1689), pow2 periods only, no eager fill.  In the
non-accepting branch it reads the OLDEST slot's score with a strict ``>`` (:1778-1787) and
overwrites the NEWEST slot (:1461); with all-zero scores (the regime of the reference's own tests,
cascade/models/test.py:499-807) both implementations must agree.
"""


class SlowCacheRestated:
    def __init__(self, window_length, num_sink_tokens, max_seq_len):
        self.W, self.NS, self.S = window_length, num_sink_tokens, max_seq_len
        self.C = max_seq_len // window_length
        self.every_n = [2 ** i for i in range(self.C)]  # :1534-1538
        self.do_cache = [True] * self.C
        self.seen = 0
        self.sinks = []                   # token payloads
        self.sink_pos = [0] * self.NS
        self.keys = [None] * self.S
        self.scores = [0.0] * self.S
        self.masked = [True] * self.S
        self.stored = [0] * self.C
        self.start = [0] * self.C
        self.pos = [0] * self.S
        self.pos_ub = max_seq_len

    def _segment_pos(self, i):  # :1351-1366
        l = i * self.W
        seg = min(self.stored[i], self.W)
        for j in range(self.W):
            self.pos[l + j] = (j + (seg - self.start[i])) % seg + (self.pos_ub - seg)
        self.pos_ub -= seg

    def _append(self, i, key, score):  # :1369-1399
        s = self.start[i] + i * self.W + self.stored[i]
        self.keys[s], self.scores[s], self.masked[s] = key, score, False
        self.stored[i] += 1
        self._segment_pos(i)

    def update(self, key, score=0.0):
        """One token (cascading_cache.py:1800-1843). Returns the position list handed to the model."""
        self.seen += 1
        for i in range(self.C):  # set_cache_bools, :1680-1689
            self.do_cache[i] = (self.seen - 1 - self.NS) % self.every_n[i] == 0
        if len(self.sinks) < self.NS:  # :1811-1818
            self.sink_pos[len(self.sinks)] = len(self.sinks)
            self.sinks.append(key)
            return list(self.pos)

        # add_keys, :1711-1798
        total = sum(self.stored)
        n_do = sum(self.do_cache)
        add_to_cache = n_do * self.W > total
        eager_add = n_do * self.W == total and total < self.S
        self.pos_ub = total + 1 if (add_to_cache or eager_add) else total
        for i in range(self.C):
            l = i * self.W
            if self.do_cache[i]:
                if self.stored[i] < self.W:
                    self._append(i, key, score)
                    break
                s = self.start[i] + l  # evict_from_cache, :1402-1442
                key, self.keys[s] = self.keys[s], key
                score, self.scores[s] = self.scores[s], score
                self.start[i] = (self.start[i] + 1) % self.W
                self._segment_pos(i)
                if i + 1 > self.C - 1:
                    break
            else:
                if self.stored[i] == 0:
                    self._append(i, key, score)
                    break
                if self.scores[self.start[i] + l] > score:  # :1778-1787
                    break
                s = max(((self.start[i] - 1) % self.stored[i]) + l, 0)  # overwrite_cache, :1445-1478
                self.keys[s], self.scores[s] = key, score
                self._segment_pos(i)
                break
        return [p + self.NS for p in self.pos]  # :1823
