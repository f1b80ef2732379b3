"""The drafters that need no second model and the round's window policy (host code, no GPU): the oracle against the
reference's own known answers (crates/shadowzero-serve/src/engine.rs:2899-2942) and against the definition, then the library
against the oracle on random conversations and random sequences of rounds."""
import os
import sys

import numpy as np
import pytest

import shadow_engine_amd as sz

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import drafter as OD   # noqa: E402


def both_drafters(min_match, max_match):
    return OD.SuffixDrafter(min_match, max_match), sz.SuffixDrafter(min_match, max_match, 64)


@pytest.mark.parametrize("which", [0, 1])
def test_suffix_drafter_known_answer_of_the_reference(which):
    """engine.rs:2899-2918: the longer of two earlier occurrences wins, and a continuation behind a neural proposal."""
    d = both_drafters(4, 32)[which]
    d.extend([1, 2, 10, 11, 12, 13, 20, 21, 22, 99])
    d.extend([5, 9, 10, 11, 12, 13, 30, 31, 32, 33, 88])
    d.extend([9, 10, 11, 12, 13])
    assert d.propose(4) == ([30, 31, 32, 33], 5)
    n = len(d.hist) if which == 0 else len(d)
    assert d.propose_after([30, 31], 3) == ([32, 33, 88], 7)
    assert (len(d.hist) if which == 0 else len(d)) == n, "a question behind a proposal must not change the history"
    assert d.propose(4) == ([30, 31, 32, 33], 5)


def brute_force_propose(hist, pushed, max_k, min_m, max_match):
    """The definition without any index: the four most recent earlier ends of the tail's trigram among the pushed tokens."""
    n = len(hist)
    min_m = max(min_m, 3)
    if n < min_m + 1 or max_k == 0:
        return [], 0
    cur = n - 1
    ends = []
    for e in range(pushed - 1, 1, -1):
        if hist[e - 2] == hist[cur - 2] and hist[e - 1] == hist[cur - 1] and hist[e] == hist[cur]:
            ends.append(e)
            if len(ends) == 4:
                break
    best = (0, 0)
    for p in ends:
        if p >= cur:
            continue
        length = 0
        while length < max_match and p - length >= 0 and hist[p - length] == hist[cur - length]:
            length += 1
        if length > best[1]:
            best = (p, length)
    if best[1] < min_m:
        return [], 0
    return hist[best[0] + 1:cur + 1][:max_k], best[1]


def test_suffix_drafter_follows_its_definition_on_random_conversations():
    """Small alphabets so that trigrams repeat many times: proposals, match lengths, the tie to the most recent place, the cap
    at max_match, the overlap of a match with the tail, the four-way memory, and questions behind a proposal."""
    rng = np.random.default_rng(5)
    asked = hits = 0
    for trial in range(60):
        alphabet = int(rng.integers(2, 6))
        min_match, max_match = int(rng.integers(1, 6)), int(rng.integers(3, 12))
        o, g = both_drafters(min_match, max_match)
        hist = []
        for step in range(int(rng.integers(5, 120))):
            chunk = rng.integers(0, alphabet, int(rng.integers(1, 5))).tolist()
            hist += chunk
            o.extend(chunk), g.extend(chunk)
            max_k = int(rng.integers(0, 9))
            want = brute_force_propose(hist, len(hist), max_k, max(min_match, 3), max(max_match, max(min_match, 3)))
            assert o.propose(max_k) == want
            assert g.propose(max_k) == want, (trial, step)
            mm = int(rng.integers(3, 8))
            want = brute_force_propose(hist, len(hist), max_k, mm, max(max_match, max(min_match, 3)))
            assert o.propose(max_k, mm) == want and g.propose(max_k, mm) == want
            extra = rng.integers(0, alphabet, int(rng.integers(1, 4))).tolist()
            want = brute_force_propose(hist + extra, len(hist), max_k, max(min_match, 3), max(max_match, max(min_match, 3)))
            assert o.propose_after(extra, max_k) == want
            assert g.propose_after(extra, max_k) == want
            asked += 1
            hits += bool(want[0])
        assert len(g) == len(hist)
    assert hits > asked // 4


def test_suffix_drafter_with_many_distinct_tokens_grows_its_table():
    rng = np.random.default_rng(6)
    o, g = both_drafters(3, 16)
    text = rng.integers(0, 50000, 9000).tolist()
    o.extend(text), g.extend(text)
    again = text[4000:4040]
    o.extend(again), g.extend(again)
    want = (text[4040:4046], 16)
    assert o.propose(6) == want and g.propose(6) == want
    assert g.propose(6, 0, [text[4040]]) == (text[4041:4047], 16)


def test_the_drafter_and_policy_refuse_null_arguments():
    L = sz.lib()
    assert L.sz_suffix_drafter_extend(None, None, 0) != 0 and "null" in sz.last_error()
    assert L.sz_draft_policy_observe(None, 0, 1, 0, 0, 1.0) != 0
    assert L.sz_draft_policy_neural_k(None, 5) == 0 and L.sz_suffix_drafter_len(None) == 0


@pytest.mark.parametrize("which", [0, 1])
def test_draft_policy_known_answer_of_the_reference(which):
    """engine.rs:2920-2941: full windows deepen the neural drafter, a long match beats the neural window, empty windows make it shallow."""
    dp = (OD.DraftPolicy, sz.DraftPolicy)[which](8, 3, 0.03)
    assert dp.neural_k(100) == 3
    for _ in range(4):
        dp.observe(False, 4, 3, 0, 12.0)
    assert dp.neural_k(100) == 4
    lookup, t = dp.choose(4, 6, 16)
    assert lookup and t >= 5
    for _ in range(8):
        dp.observe(False, 4, 0, 0, 12.0)
    assert dp.neural_k(100) == 2
    assert dp.neural_k(1) == 1 and dp.neural_k(0) == 0


def test_draft_policy_closed_forms_before_and_after_observations():
    """What the formulas fix without running them: the priors, the cost curve moved from one observed size to the others, the
    running means' first value and their decay."""
    o = OD.DraftPolicy(8, 3, 0.03)
    g = sz.DraftPolicy(8, 3, 0.03)
    st = g.state()
    assert np.allclose(st["lookup_rate"], [0.75, 0.88, 0.93, 0.96]) and np.allclose(st["chain_rate"], [0.45, 0.65, 0.80, 0.90])
    assert np.allclose(st["cost_ms"], OD.SHAPE[1:]) and st["accept_ema"] == 0.65 and st["rounds"] == 0
    for p in (o, g):
        p.observe(True, 5, 4, 13, 20.5)       # a lookup round of 5 rows: all 4 drafts kept, 20.5 ms
    st = g.state()
    assert st["cost_ms"][4] == 20.5 and np.allclose(st["cost_ms"], [20.5 * OD.SHAPE[t] / OD.SHAPE[5] for t in range(1, 9)])
    assert np.isclose(st["lookup_rate"][2], (4 + 4 * 0.93) / (4 + 0 + 4)) and st["lookup_rate"][0] == 0.75
    for p in (o, g):
        p.observe(True, 5, 1, 13, 30.5)       # the second: one draft kept of four
    st = g.state()
    assert np.isclose(st["cost_ms"][4], 0.9 * 20.5 + 0.1 * 30.5)
    assert np.isclose(st["lookup_rate"][2], (0.97 * 4 + 1 + 4 * 0.93) / (0.97 * 4 + 1 + 1 + 4))
    assert np.isclose(o.lookup_rate(13), st["lookup_rate"][2], rtol=0, atol=1e-15)
    # an unchained neural round feeds the acceptance mean: 0.75 * 0.65 + 0.25 * 2/3
    for p in (o, g):
        p.observe(False, 4, 2, 0, 15.0)
    assert np.isclose(g.state()["accept_ema"], 0.75 * 0.65 + 0.25 * 2 / 3) and o.accept_ema == g.state()["accept_ema"]


def test_draft_policy_matches_the_oracle_over_random_rounds():
    rng = np.random.default_rng(9)
    for trial in range(25):
        max_t, base, margin = int(rng.integers(1, 10)), int(rng.integers(1, 9)), float(rng.choice([0.0, 0.03, 0.2]))
        o, g = OD.DraftPolicy(max_t, base, margin), sz.DraftPolicy(max_t, base, margin)
        for step in range(400):
            kind = rng.integers(0, 6)
            t = int(rng.integers(0, 11))
            ml = int(rng.integers(0, 40))
            if kind == 0:
                acc = int(rng.integers(0, max(t, 1) + 1))
                ms = float(rng.choice([0.0, rng.uniform(5, 60)]))
                lk = bool(rng.integers(0, 2))
                o.observe(lk, t, acc, ml, ms), g.observe(lk, t, acc, ml, ms)
            elif kind == 1:
                kc, acc = int(rng.integers(0, 6)), int(rng.integers(0, 10))
                ms = float(rng.uniform(5, 60))
                o.observe_chain(t, kc, acc, ml, ms), g.observe_chain(t, kc, acc, ml, ms)
            elif kind == 2:
                k = int(rng.integers(0, 10))
                assert o.choose(t, k, ml) == g.choose(t, k, ml), (trial, step)
            elif kind == 3:
                pn, k = float(rng.uniform(-0.2, 1.2)), int(rng.integers(0, 10))
                assert o.chain(t, pn, k, ml) == g.chain(t, pn, k, ml), (trial, step)
            elif kind == 4:
                rem = int(rng.integers(0, 12))
                assert o.neural_k(rem) == g.neural_k(rem)
            else:
                # a long quiet stretch makes the sizes stale, which the choice then probes again
                for _ in range(int(rng.integers(0, 350))):
                    o.observe(False, 2, 1, 0, 0.0), g.observe(False, 2, 1, 0, 0.0)
        st = g.state()
        assert st["accept_ema"] == o.accept_ema and st["rounds"] == o.rounds
        assert np.array_equal(st["cost_ms"], [o.cost_ms(t) for t in range(1, 9)])
        assert np.array_equal(st["lookup_rate"], [o.lookup_rate(m) for m in (3, 6, 12, 24)])
        assert np.array_equal(st["chain_rate"], [o.chain_rate(m) for m in (3, 6, 12, 24)])
