// The host side of a speculative round that sits in front of the verify step: where the drafts come from when no second
// model is asked.  Two pieces of crates/shadowzero-serve/src/engine.rs, restated as plain C entry points:
//   the suffix drafter (engine.rs:844-1015): every trigram of the conversation remembers the last four places it ended;
//     the draft is what followed the longest earlier occurrence of the conversation's tail, and a continuation can be asked
//     for behind a neural drafter's proposal without touching the index;
//   the draft policy (engine.rs:1017-1311): running estimates of what a round of t rows costs and of how many drafts are
//     kept, from which it decides between the neural window and a lookup window, how many looked-up tokens to chain behind a
//     neural draft, and how deep the neural drafter should go.
// Host code only; nothing here touches the GPU.  The numbers (priors, decay, shape of the cost curve) are the reference's,
// since a policy that decides differently is a different policy.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <vector>

#include "sz_internal.hpp"

namespace {

constexpr uint32_t WAYS = 4;       // SUFFIX_WAYS, engine.rs:841
constexpr uint32_t MAX_T = 8;      // DP_MAX_T = MAX_VERIFY (session.rs), engine.rs:1017
constexpr uint32_t BUCKETS = 4;    // match lengths < 6, 6..11, 12..23, >= 24 (engine.rs:1086-1096)
constexpr double SHAPE[MAX_T + 1] = {0.0, 1.0, 1.35, 1.70, 2.05, 2.45, 2.85, 3.25, 3.60};   // engine.rs:1019
constexpr double COST_ALPHA = 0.10, TOK_ALPHA = 0.05, DECAY = 0.97, PRIOR_N = 4.0, PROBES = 3.0, STALE_ROUNDS = 300.0;
constexpr double PRIOR_Q[BUCKETS] = {0.75, 0.88, 0.93, 0.96}, CHAIN_PRIOR[BUCKETS] = {0.45, 0.65, 0.80, 0.90};

// A trigram's record.  The reference keys its table by a 64-bit hash of the three tokens and takes equal hashes for equal
// trigrams; here the tokens themselves are the key, so two trigrams never share a record.
struct Trigram {
    uint32_t a = 0, b = 0, c = 0;
    uint32_t used = 0;             // how many of ends[] are set (0: the slot is free)
    uint32_t ends[WAYS] = {};      // positions of the trigram's last token, most recent first
};

uint64_t spread(uint32_t a, uint32_t b, uint32_t c) {
    uint64_t h = (uint64_t) a * 0x9E3779B97F4A7C15ull;
    h ^= ((uint64_t) b << 21) | (b >> 11);
    h *= 0xD6E8FEB86659FD93ull;
    h ^= (uint64_t) c * 0xA24BAED4963EE407ull;
    return h ^ (h >> 29);
}

uint32_t bucket_of(uint32_t match_len) { return match_len < 6 ? 0 : match_len < 12 ? 1 : match_len < 24 ? 2 : 3; }

}   // namespace

struct sz_suffix_drafter {
    uint32_t min_match, max_match;
    std::vector<uint32_t> hist;
    std::vector<Trigram> table;    // open addressing, a power of two of slots, grown when half full
    uint64_t filled = 0;

    Trigram* slot(uint32_t a, uint32_t b, uint32_t c, bool make) {
        const uint64_t mask = table.size() - 1;
        for (uint64_t i = spread(a, b, c) & mask;; i = (i + 1) & mask) {
            Trigram& t = table[i];
            if (t.used == 0) {
                if (!make) return nullptr;
                t.a = a, t.b = b, t.c = c;
                filled++;
                return &t;
            }
            if (t.a == a && t.b == b && t.c == c) return &t;
        }
    }
    void grow() {
        std::vector<Trigram> old(table.size() * 2);
        old.swap(table);
        filled = 0;
        for (const Trigram& t : old)
            if (t.used) {
                Trigram* n = slot(t.a, t.b, t.c, true);
                *n = t;
            }
    }
    void push(uint32_t token) {
        hist.push_back(token);
        const size_t end = hist.size() - 1;
        if (end < 2) return;
        if (2 * (filled + 1) > table.size()) grow();
        Trigram* t = slot(hist[end - 2], hist[end - 1], hist[end], true);
        for (uint32_t w = WAYS - 1; w > 0; w--) t->ends[w] = t->ends[w - 1];
        t->ends[0] = (uint32_t) end;
        if (t->used < WAYS) t->used++;
    }
    // engine.rs:954-990 on hist[0..n): the continuation of the longest earlier occurrence of the tail
    void propose(size_t n, uint32_t max_k, uint32_t min_m, std::vector<uint32_t>& out, uint32_t& match_len) {
        out.clear();
        match_len = 0;
        min_m = std::max(min_m, 3u);
        if (n < (size_t) min_m + 1 || max_k == 0) return;
        const size_t cur = n - 1;
        const Trigram* t = slot(hist[cur - 2], hist[cur - 1], hist[cur], false);
        if (!t) return;
        size_t best_end = 0, best_len = 0;
        for (uint32_t w = 0; w < t->used; w++) {
            const size_t p = t->ends[w];
            if (p >= cur) continue;
            size_t len = 0;
            while (len < max_match && len <= p && hist[p - len] == hist[cur - len]) len++;
            if (len > best_len) best_len = len, best_end = p;      // the more recent place keeps a tie
        }
        if (best_len < min_m) return;
        for (size_t q = best_end + 1; q <= cur && out.size() < max_k; q++) out.push_back(hist[q]);
        match_len = (uint32_t) best_len;
    }
};

struct sz_draft_policy {
    uint32_t max_t, base_spec;
    double margin;
    double cost[MAX_T + 1] = {}, cost_n[MAX_T + 1] = {}, tok[MAX_T + 1] = {}, tok_n[MAX_T + 1] = {}, last[MAX_T + 1] = {};
    double ok[BUCKETS] = {}, bad[BUCKETS] = {}, cok[BUCKETS] = {}, cbad[BUCKETS] = {};
    double rounds = 0.0, accept_ema = 0.65;
    uint32_t full_streak = 0, zero_streak = 0;

    static uint32_t clamp_t(uint32_t t) { return std::min(std::max(t, 1u), MAX_T); }
    double lookup_rate(uint32_t ml) const {
        const uint32_t b = bucket_of(ml);
        return (ok[b] + PRIOR_N * PRIOR_Q[b]) / (ok[b] + bad[b] + PRIOR_N);
    }
    double chain_rate(uint32_t ml) const {
        const uint32_t b = bucket_of(ml);
        return (cok[b] + PRIOR_N * CHAIN_PRIOR[b]) / (cok[b] + cbad[b] + PRIOR_N);
    }
    // what a round of t rows costs: its own running mean, else the other sizes' means moved along the shape curve
    double cost_ms(uint32_t t) const {
        t = clamp_t(t);
        if (cost_n[t] > 0.0) return cost[t];
        double num = 0.0, den = 0.0;
        for (uint32_t u = 1; u <= MAX_T; u++)
            if (cost_n[u] > 0.0) {
                const double w = std::min(cost_n[u], 20.0);
                num += w * cost[u] * SHAPE[t] / SHAPE[u];
                den += w;
            }
        return den > 0.0 ? num / den : SHAPE[t];
    }
    bool stale(uint32_t t) const { return cost_n[t] > 0.0 && rounds - last[t] > STALE_ROUNDS; }
    double neural_tokens(uint32_t t) const {
        t = clamp_t(t);
        return tok_n[t] > 0.0 ? tok[t] : 1.0 + 0.70 * (double) (t - 1);
    }
    void note_cost(uint32_t t, double round_ms) {
        if (round_ms > 0.0) {
            cost[t] = cost_n[t] > 0.0 ? (1.0 - COST_ALPHA) * cost[t] + COST_ALPHA * round_ms : round_ms;
            cost_n[t] += 1.0;
            last[t] = rounds;
        }
        rounds += 1.0;
    }
    void note_streak(uint32_t drafted, uint32_t accepted) {
        if (drafted == 0) return;
        const double rate = (double) std::min(accepted, drafted) / (double) drafted;
        accept_ema = 0.75 * accept_ema + 0.25 * rate;
        if (accepted >= drafted) full_streak++, zero_streak = 0;
        else if (accepted == 0) zero_streak++, full_streak = 0;
        else full_streak = zero_streak = 0;
    }
    void note_tokens(uint32_t t, uint32_t accepted) {
        const double got = (double) accepted + 1.0;
        tok[t] = tok_n[t] > 0.0 ? (1.0 - TOK_ALPHA) * tok[t] + TOK_ALPHA * got : got;
        tok_n[t] += 1.0;
    }
};

extern "C" {

sz_suffix_drafter* sz_suffix_drafter_new(uint32_t min_match, uint32_t max_match, uint32_t capacity_tokens) {
    sz::clear_error();
    auto* d = new sz_suffix_drafter();
    d->min_match = std::max(min_match, 3u);
    d->max_match = std::max(max_match, d->min_match);
    d->hist.reserve(capacity_tokens);
    uint64_t slots = 2048;
    while (slots < 2ull * std::max(capacity_tokens, 1024u)) slots *= 2;
    d->table.resize(slots);
    return d;
}

void sz_suffix_drafter_free(sz_suffix_drafter* d) { delete d; }

int32_t sz_suffix_drafter_extend(sz_suffix_drafter* d, const uint32_t* tokens, uint32_t n) {
    sz::clear_error();
    if (!d || (n && !tokens)) return sz::fail("sz_suffix_drafter_extend: null argument");
    if (d->hist.size() + n > 0xffffffffull) return sz::fail("sz_suffix_drafter_extend: more than 2^32 tokens");
    for (uint32_t i = 0; i < n; i++) d->push(tokens[i]);
    return 0;
}

uint64_t sz_suffix_drafter_len(const sz_suffix_drafter* d) { return d ? d->hist.size() : 0; }

int32_t sz_suffix_drafter_propose(sz_suffix_drafter* d, const uint32_t* extra, uint32_t n_extra, uint32_t max_k, uint32_t min_match, uint32_t* drafts,
                                  uint32_t* n_drafts, uint32_t* match_len) {
    sz::clear_error();
    if (!d || !n_drafts || !match_len || (n_extra && !extra) || (max_k && !drafts)) return sz::fail("sz_suffix_drafter_propose: null argument");
    const size_t n0 = d->hist.size();
    // the proposal of a neural drafter goes behind the history for the question and comes off again: the index only
    // ever holds what was said (engine.rs:998-1014)
    d->hist.insert(d->hist.end(), extra, extra + n_extra);
    std::vector<uint32_t> out;
    d->propose(d->hist.size(), max_k, min_match ? min_match : d->min_match, out, *match_len);
    d->hist.resize(n0);
    *n_drafts = (uint32_t) out.size();
    std::copy(out.begin(), out.end(), drafts);
    return 0;
}

sz_draft_policy* sz_draft_policy_new(uint32_t max_t, uint32_t base_spec, double margin) {
    sz::clear_error();
    auto* p = new sz_draft_policy();
    p->max_t = std::min(std::max(max_t, 1u), MAX_T);
    p->base_spec = std::min(std::max(base_spec, 1u), MAX_T - 1);
    p->margin = margin;
    return p;
}

void sz_draft_policy_free(sz_draft_policy* p) { delete p; }

uint32_t sz_draft_policy_neural_k(const sz_draft_policy* p, uint32_t rem_tokens) {
    if (!p) return 0;
    const uint32_t max_k = std::min(p->max_t - 1, rem_tokens);
    if (max_k == 0) return 0;
    uint32_t k = p->base_spec;
    if (p->full_streak >= 2 && p->accept_ema >= 0.75) k = std::min(p->base_spec + 1, p->max_t - 1);
    else if (p->zero_streak >= 3 && p->accept_ema < 0.25) k = std::min(2u, p->base_spec);
    return std::min(k, max_k);
}

int32_t sz_draft_policy_choose(const sz_draft_policy* p, uint32_t t_neural, uint32_t lookup_k, uint32_t match_len, int32_t* lookup, uint32_t* t) {
    sz::clear_error();
    if (!p || !lookup || !t) return sz::fail("sz_draft_policy_choose: null argument");
    *lookup = 0;
    *t = std::min(std::max(t_neural, 1u), p->max_t);
    if (lookup_k == 0) return 0;
    const double base = p->neural_tokens(*t) / p->cost_ms(*t);
    const double q = p->lookup_rate(match_len);
    // expected tokens of a window of k looked-up drafts: 1 + q + q^2 + .. + q^k, per millisecond of a round of k + 1 rows
    double e = 1.0, qi = 1.0, best = 0.0;
    uint32_t best_t = 0;
    const uint32_t k_lim = std::min(lookup_k, p->max_t - 1);
    for (uint32_t k = 1; k <= k_lim; k++) {
        qi *= q;
        e += qi;
        const double r = e / p->cost_ms(k + 1);
        if (r > best) best = r, best_t = k + 1;
    }
    const uint32_t t_full = k_lim + 1;
    if (best_t > 0 && best > base * (1.0 + p->margin)) {
        *lookup = 1;
        *t = (best_t < t_full && q >= 0.85 && p->stale(t_full)) ? t_full : best_t;   // a size not seen for long is tried again
        return 0;
    }
    if (t_full > *t && (p->cost_n[t_full] < PROBES || p->stale(t_full)) && q >= 0.85) {
        *lookup = 1;
        *t = t_full;
    }
    return 0;
}

uint32_t sz_draft_policy_chain(const sz_draft_policy* p, uint32_t t_neural, double p_neural, uint32_t k_avail, uint32_t match_len) {
    if (!p) return 0;
    t_neural = std::min(std::max(t_neural, 1u), p->max_t);
    const uint32_t kmax = std::min(k_avail, p->max_t - t_neural);
    if (kmax == 0) return 0;
    const double e0 = p->neural_tokens(t_neural), base = e0 / p->cost_ms(t_neural), c = p->chain_rate(match_len);
    p_neural = std::min(std::max(p_neural, 0.0), 1.0);
    double gain = 0.0, ci = 1.0, best = 0.0;
    uint32_t best_k = 0;
    for (uint32_t k = 1; k <= kmax; k++) {
        ci *= c;
        gain += ci;
        const double r = (e0 + p_neural * gain) / p->cost_ms(t_neural + k);
        if (r > best) best = r, best_k = k;
    }
    const uint32_t t_full = t_neural + kmax;
    if (best_k > 0 && best > base * (1.0 + p->margin)) return (best_k < kmax && p_neural * c >= 0.60 && p->stale(t_full)) ? kmax : best_k;
    if ((p->cost_n[t_full] < PROBES || p->stale(t_full)) && p_neural * c >= 0.60) return kmax;
    return 0;
}

int32_t sz_draft_policy_observe(sz_draft_policy* p, int32_t lookup, uint32_t t, uint32_t accepted, uint32_t match_len, double round_ms) {
    sz::clear_error();
    if (!p) return sz::fail("sz_draft_policy_observe: null policy");
    t = sz_draft_policy::clamp_t(t);
    p->note_cost(t, round_ms);
    if (lookup) {
        const uint32_t b = bucket_of(match_len);
        p->ok[b] = DECAY * p->ok[b] + (double) accepted;
        p->bad[b] = DECAY * p->bad[b] + (accepted < t - 1 ? 1.0 : 0.0);
    } else {
        p->note_streak(t - 1, accepted);
        p->note_tokens(t, accepted);
    }
    return 0;
}

int32_t sz_draft_policy_observe_chain(sz_draft_policy* p, uint32_t t_neural, uint32_t k_chain, uint32_t accepted, uint32_t match_len, double round_ms) {
    sz::clear_error();
    if (!p) return sz::fail("sz_draft_policy_observe_chain: null policy");
    t_neural = sz_draft_policy::clamp_t(t_neural);
    p->note_cost(sz_draft_policy::clamp_t(t_neural + k_chain), round_ms);
    const uint32_t drafted = t_neural - 1, kept = std::min(accepted, drafted);
    p->note_streak(drafted, kept);
    p->note_tokens(t_neural, kept);
    if (accepted < drafted) return 0;            // the chain was never reached
    const uint32_t b = bucket_of(match_len), got = accepted - drafted;
    p->cok[b] = DECAY * p->cok[b] + (double) got;
    p->cbad[b] = DECAY * p->cbad[b] + (got < k_chain ? 1.0 : 0.0);
    return 0;
}

int32_t sz_draft_policy_state(const sz_draft_policy* p, double* accept_ema, double* rounds, double* cost_ms8, double* lookup_rate4, double* chain_rate4) {
    sz::clear_error();
    if (!p) return sz::fail("sz_draft_policy_state: null policy");
    if (accept_ema) *accept_ema = p->accept_ema;
    if (rounds) *rounds = p->rounds;
    if (cost_ms8)
        for (uint32_t t = 1; t <= MAX_T; t++) cost_ms8[t - 1] = p->cost_ms(t);
    static const uint32_t probe[BUCKETS] = {3, 6, 12, 24};
    for (uint32_t b = 0; b < BUCKETS; b++) {
        if (lookup_rate4) lookup_rate4[b] = p->lookup_rate(probe[b]);
        if (chain_rate4) chain_rate4[b] = p->chain_rate(probe[b]);
    }
    return 0;
}

}   // extern "C"
