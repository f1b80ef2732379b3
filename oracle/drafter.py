"""CPU restatement of the reference's draft sources that need no second model, for the tests only (test infrastructure: the
library never loads it).

  suffix drafter   crates/shadowzero-serve/src/engine.rs:844-1015 (SuffixDrafter: push, propose_with_min, propose_after)
  draft policy     crates/shadowzero-serve/src/engine.rs:1017-1311 (DraftPolicy: neural_k, choose, chain, observe, observe_chain)

The suffix drafter is stated by its definition, with a scan instead of the reference's hash table (which takes two trigrams
with the same 64-bit hash for one; the definition does not): the candidates are the four most recent places where the
tail's last trigram ended among the tokens that were pushed, the winner is the candidate with the longest match backwards
(at most max_match tokens; the more recent one on a tie), and the draft is what followed it.

Pinned by the reference's own tests of the two (engine.rs:2899-2942), asserted on this file in tests/test_drafter.py, and by
closed forms where the policy has them (priors before any observation, the cost curve's extrapolation).
"""

WAYS = 4
MAX_T = 8
SHAPE = [0.0, 1.0, 1.35, 1.70, 2.05, 2.45, 2.85, 3.25, 3.60]
COST_ALPHA, TOK_ALPHA, DECAY, PRIOR_N, PROBES, STALE_ROUNDS = 0.10, 0.05, 0.97, 4.0, 3.0, 300.0
PRIOR_Q = [0.75, 0.88, 0.93, 0.96]
CHAIN_PRIOR = [0.45, 0.65, 0.80, 0.90]


class SuffixDrafter:
    def __init__(self, min_match, max_match, capacity_tokens=0):
        self.min_match = max(min_match, 3)                       # engine.rs:870
        self.max_match = max(max_match, self.min_match)
        self.hist = []

    def extend(self, tokens):
        self.hist.extend(int(t) for t in tokens)

    def _propose(self, seq, pushed, max_k, min_match):
        min_m = max(min_match, 3)                                # engine.rs:955
        n = len(seq)
        if n < min_m + 1 or max_k == 0:
            return [], 0
        cur = n - 1
        tri = seq[cur - 2:cur + 1]
        # the table holds the last WAYS ends of every trigram among the pushed tokens (engine.rs:929-945), the tail's own
        # end included when it was pushed
        ends = [e for e in range(2, pushed) if seq[e - 2:e + 1] == tri][-WAYS:][::-1]
        best_end, best_len = 0, 0
        for p in ends:
            if p >= cur:
                continue
            length = 0
            while length < self.max_match and length <= p and seq[p - length] == seq[cur - length]:
                length += 1
            if length > best_len:
                best_end, best_len = p, length
        if best_len < min_m:
            return [], 0
        return seq[best_end + 1:min(best_end + 1 + max_k, cur + 1)], best_len

    def propose(self, max_k, min_match=None):
        return self._propose(self.hist, len(self.hist), max_k, self.min_match if min_match is None else min_match)

    def propose_after(self, extra, max_k):
        """engine.rs:998-1014: the question is asked of history + extra, the index stays that of the history."""
        extra = [int(t) for t in extra]
        if not extra:
            return self.propose(max_k)
        if max_k == 0:
            return [], 0
        return self._propose(self.hist + extra, len(self.hist), max_k, self.min_match)


def bucket(match_len):
    return 0 if match_len < 6 else 1 if match_len < 12 else 2 if match_len < 24 else 3


class DraftPolicy:
    def __init__(self, max_t, base_spec, margin):
        self.max_t = min(max(max_t, 1), MAX_T)
        self.base_spec = min(max(base_spec, 1), MAX_T - 1)
        self.margin = margin
        z = [0.0] * (MAX_T + 1)
        self.cost, self.cost_n, self.tok, self.tok_n, self.last = z[:], z[:], z[:], z[:], z[:]
        self.ok, self.bad, self.cok, self.cbad = [0.0] * 4, [0.0] * 4, [0.0] * 4, [0.0] * 4
        self.rounds, self.accept_ema, self.full_streak, self.zero_streak = 0.0, 0.65, 0, 0

    def lookup_rate(self, ml):
        b = bucket(ml)
        return (self.ok[b] + PRIOR_N * PRIOR_Q[b]) / (self.ok[b] + self.bad[b] + PRIOR_N)

    def chain_rate(self, ml):
        b = bucket(ml)
        return (self.cok[b] + PRIOR_N * CHAIN_PRIOR[b]) / (self.cok[b] + self.cbad[b] + PRIOR_N)

    def cost_ms(self, t):
        t = min(max(t, 1), MAX_T)
        if self.cost_n[t] > 0.0:
            return self.cost[t]
        num = den = 0.0
        for u in range(1, MAX_T + 1):
            if self.cost_n[u] > 0.0:
                w = min(self.cost_n[u], 20.0)
                num += w * self.cost[u] * SHAPE[t] / SHAPE[u]
                den += w
        return num / den if den > 0.0 else SHAPE[t]

    def stale(self, t):
        return self.cost_n[t] > 0.0 and self.rounds - self.last[t] > STALE_ROUNDS

    def neural_tokens(self, t):
        t = min(max(t, 1), MAX_T)
        return self.tok[t] if self.tok_n[t] > 0.0 else 1.0 + 0.70 * (t - 1)

    def neural_k(self, rem):
        max_k = min(self.max_t - 1, rem)
        if max_k == 0:
            return 0
        k = self.base_spec
        if self.full_streak >= 2 and self.accept_ema >= 0.75:
            k = min(self.base_spec + 1, self.max_t - 1)
        elif self.zero_streak >= 3 and self.accept_ema < 0.25:
            k = min(2, self.base_spec)
        return min(k, max_k)

    def choose(self, t_neural, lookup_k, match_len):
        """(lookup, t)"""
        t = min(max(t_neural, 1), self.max_t)
        if lookup_k == 0:
            return False, t
        base = self.neural_tokens(t) / self.cost_ms(t)
        q = self.lookup_rate(match_len)
        e, qi, best, best_t = 1.0, 1.0, 0.0, 0
        k_lim = min(lookup_k, self.max_t - 1)
        for k in range(1, k_lim + 1):
            qi *= q
            e += qi
            r = e / self.cost_ms(k + 1)
            if r > best:
                best, best_t = r, k + 1
        t_full = k_lim + 1
        if best_t > 0 and best > base * (1.0 + self.margin):
            if best_t < t_full and q >= 0.85 and self.stale(t_full):
                return True, t_full
            return True, best_t
        if t_full > t and (self.cost_n[t_full] < PROBES or self.stale(t_full)) and q >= 0.85:
            return True, t_full
        return False, t

    def chain(self, t_neural, p_neural, k_avail, match_len):
        t_neural = min(max(t_neural, 1), self.max_t)
        kmax = min(k_avail, self.max_t - t_neural)
        if kmax == 0:
            return 0
        e0 = self.neural_tokens(t_neural)
        base = e0 / self.cost_ms(t_neural)
        c = self.chain_rate(match_len)
        p_neural = min(max(p_neural, 0.0), 1.0)
        gain, ci, best, best_k = 0.0, 1.0, 0.0, 0
        for k in range(1, kmax + 1):
            ci *= c
            gain += ci
            r = (e0 + p_neural * gain) / self.cost_ms(t_neural + k)
            if r > best:
                best, best_k = r, k
        t_full = t_neural + kmax
        if best_k > 0 and best > base * (1.0 + self.margin):
            if best_k < kmax and p_neural * c >= 0.60 and self.stale(t_full):
                return kmax
            return best_k
        if (self.cost_n[t_full] < PROBES or self.stale(t_full)) and p_neural * c >= 0.60:
            return kmax
        return 0

    def _note_cost(self, t, round_ms):
        if round_ms > 0.0:
            self.cost[t] = (1.0 - COST_ALPHA) * self.cost[t] + COST_ALPHA * round_ms if self.cost_n[t] > 0.0 else round_ms
            self.cost_n[t] += 1.0
            self.last[t] = self.rounds
        self.rounds += 1.0

    def _note_streak(self, drafted, accepted):
        if drafted == 0:
            return
        self.accept_ema = 0.75 * self.accept_ema + 0.25 * (min(accepted, drafted) / drafted)
        if accepted >= drafted:
            self.full_streak, self.zero_streak = self.full_streak + 1, 0
        elif accepted == 0:
            self.zero_streak, self.full_streak = self.zero_streak + 1, 0
        else:
            self.full_streak = self.zero_streak = 0

    def _note_tokens(self, t, accepted):
        got = accepted + 1.0
        self.tok[t] = (1.0 - TOK_ALPHA) * self.tok[t] + TOK_ALPHA * got if self.tok_n[t] > 0.0 else got
        self.tok_n[t] += 1.0

    def observe(self, lookup, t, accepted, match_len, round_ms):
        t = min(max(t, 1), MAX_T)
        self._note_cost(t, round_ms)
        if lookup:
            b = bucket(match_len)
            self.ok[b] = DECAY * self.ok[b] + accepted
            self.bad[b] = DECAY * self.bad[b] + (1.0 if accepted < t - 1 else 0.0)
        else:
            self._note_streak(t - 1, accepted)
            self._note_tokens(t, accepted)

    def observe_chain(self, t_neural, k_chain, accepted, match_len, round_ms):
        t_neural = min(max(t_neural, 1), MAX_T)
        self._note_cost(min(max(t_neural + k_chain, 1), MAX_T), round_ms)
        drafted = t_neural - 1
        kept = min(accepted, drafted)
        self._note_streak(drafted, kept)
        self._note_tokens(t_neural, kept)
        if accepted < drafted:
            return
        b = bucket(match_len)
        got = accepted - drafted
        self.cok[b] = DECAY * self.cok[b] + got
        self.cbad[b] = DECAY * self.cbad[b] + (1.0 if got < k_chain else 0.0)
