"""Pins the oracle's TextGen restatement (text_gen.cpp:14-209).

grad.cpp has no test and no stored vector for these functions and its sampler's
RNG cannot be seeded, so they are pinned by hand-derived cases (expected values
written out, not recomputed by the same formula), by the loop-count rules read
off the source, and by brute force against a float64 set-based restatement on
tiny vocabularies.  The reference binary's exact streams remain unpinned.
"""
import math

import numpy as np
import pytest

import oracle_lib as O
from gradhip import synth
from helpers import make_pair

LN = [math.log(1.0), math.log(2.0), math.log(3.0), math.log(4.0)]  # softmax -> .1 .2 .3 .4


def test_penalty_once_per_occurrence_in_window():
    # token 0 twice, token 1 once, penalty 2: 2.0 -> 0.5, -1.0 -> -2.0 (text_gen.cpp:23-30)
    out = O.logits_with_penalty([2.0, -1.0, 4.0], [0, 0, 1], 2.0)
    assert out.tolist() == [0.5, -2.0, 4.0]
    # exactly 0 counts as "not > 0": multiplied
    assert O.logits_with_penalty([0.0, 1.0], [0], 3.0).tolist() == [0.0, 1.0]
    # penalty 1.0 is a no-op even for repeated tokens
    assert O.logits_with_penalty([2.0, -1.0], [0, 0, 1, 1], 1.0).tolist() == [2.0, -1.0]


def test_penalty_window_is_the_last_50_tokens():
    toks = [2] * 5 + [1] * 55          # the 2s sit outside the last 50
    out = O.logits_with_penalty([8.0, 2.0 ** 60, 8.0], toks, 2.0)
    assert out[2] == 8.0 and out[0] == 8.0
    assert out[1] == 2.0 ** 10         # 50 halvings of 2^60
    toks = [2] + [1] * 49              # the 2 is the 50th from the end: inside
    assert O.logits_with_penalty([8.0, 1.0, 8.0], toks, 2.0)[2] == 4.0


def test_argmax_takes_the_first_of_equal_maxima():
    assert O.argmax_first([1.0, 5.0, 5.0, 2.0]) == 1
    assert O.argmax_first([7.0, 7.0, 7.0]) == 0
    assert O.argmax_first([-3.0, -1.0, -2.0]) == 1


def test_plain_sampling_walks_the_cdf_in_index_order():
    # probs .1 .2 .3 .4 -> cdf .1 .3 .6 1.0
    for u, want in [(0.0, 0), (0.05, 0), (0.15, 1), (0.29, 1), (0.31, 2), (0.59, 2), (0.61, 3), (0.999, 3)]:
        assert O.sample_from_logits(LN, u=u) == want
    _, p = O.sample_from_logits(LN, u=0.5, want_probs=True)
    assert np.allclose(p, [0.1, 0.2, 0.3, 0.4], atol=1e-7)


def test_temperature_divides_the_logits():
    # T = 0.5 squares the odds: 1 4 9 16 / 30
    _, p = O.sample_from_logits(LN, temperature=0.5, u=0.5, want_probs=True)
    assert np.allclose(p, np.array([1, 4, 9, 16]) / 30.0, atol=1e-6)


def test_top_k_keeps_the_k_largest_and_ties_at_the_threshold():
    _, p = O.sample_from_logits(LN, top_k=2, u=0.5, want_probs=True)
    assert np.allclose(p, [0, 0, 3 / 7, 4 / 7], atol=1e-7)
    assert O.sample_from_logits(LN, top_k=2, u=0.42) == 2
    assert O.sample_from_logits(LN, top_k=2, u=0.44) == 3
    # three equal maxima with k = 2: the threshold is 1.0 and all three survive (text_gen.cpp:148-153)
    _, p = O.sample_from_logits([1.0, 1.0, 0.0, 1.0], top_k=2, u=0.5, want_probs=True)
    assert np.allclose(p, [1 / 3, 1 / 3, 0, 1 / 3], atol=1e-7)
    # k >= V and k = 0 switch the filter off
    for k in (0, 4, 9):
        _, p = O.sample_from_logits(LN, top_k=k, u=0.5, want_probs=True)
        assert np.allclose(p, [0.1, 0.2, 0.3, 0.4], atol=1e-7)
    # top_k = 1 is `grad chat --greedy` (chat.cpp:42-44): always the arg-max
    for u in (1e-6, 0.3, 0.99):
        assert O.sample_from_logits([0.3, 2.0, -1.0, 1.9], top_k=1, u=u) == 1
    # a draw of exactly 0 satisfies `u <= cumulative` at index 0 even when p[0] == 0
    # (text_gen.cpp:202-206): the walk returns 0
    assert O.sample_from_logits([0.3, 2.0, -1.0, 1.9], top_k=1, u=0.0) == 0


def test_top_p_cuts_after_the_entry_that_reaches_p():
    # sorted .4 .3 .2 .1; p = 0.5 is reached at .3 -> keep {.3, .4}, renormalise
    _, p = O.sample_from_logits(LN, top_p=0.5, u=0.5, want_probs=True)
    assert np.allclose(p, [0, 0, 3 / 7, 4 / 7], atol=1e-7)
    # p = 0.35 is reached by the first entry alone
    _, p = O.sample_from_logits(LN, top_p=0.35, u=0.5, want_probs=True)
    assert np.allclose(p, [0, 0, 0, 1.0], atol=1e-7)
    # ties with the cutoff value survive: .25 x4, p = 0.3 -> cutoff .25 keeps all
    _, p = O.sample_from_logits([0.0] * 4, top_p=0.3, u=0.5, want_probs=True)
    assert np.allclose(p, [0.25] * 4, atol=1e-7)
    # top_p = 1 is off
    _, p = O.sample_from_logits(LN, top_p=1.0, u=0.5, want_probs=True)
    assert np.allclose(p, [0.1, 0.2, 0.3, 0.4], atol=1e-7)


def test_top_p_never_reached_keeps_only_the_maximum():
    # If rounding leaves the sorted cumulative sum below top_p, cutoff_idx stays 0
    # and only entries >= the largest probability survive (text_gen.cpp:167-177).
    top_p = float(np.nextafter(np.float32(1.0), np.float32(0.0)))
    rng = np.random.default_rng(0)
    found = 0
    for _ in range(4000):
        lg = rng.normal(0, 2, 12).astype(np.float32)
        # the softmax as the checker computed it; the sorted running sum is plain
        # fp32 addition, reproducible here
        _, p = O.sample_from_logits(lg, u=0.5, want_probs=True)
        c = np.float32(0)
        for v in np.sort(p)[::-1]:
            c = np.float32(c + v)
        if c < np.float32(top_p):
            found += 1
            for u in (0.01, 0.5, 0.97):
                assert O.sample_from_logits(lg, top_p=top_p, u=u) == int(np.argmax(lg))
            if found >= 5:
                break
    assert found >= 1


def _sample64(logits, T, k, p_nuc, u):
    """Float64, set-based statement of the sampler's documented behaviour."""
    z = np.asarray(logits, np.float64) / T
    V = len(z)
    keep = np.ones(V, bool)
    if 0 < k < V:
        kth = np.sort(z)[::-1][k - 1]
        keep = z >= kth
    e = np.where(keep, np.exp(z - z[keep].max()), 0.0)
    pr = e / e.sum()
    if p_nuc < 1.0:
        order = np.argsort(-pr, kind="stable")
        csum = np.cumsum(pr[order])
        hit = np.nonzero(csum >= p_nuc)[0]
        cutoff = pr[order[hit[0]]] if len(hit) else pr[order[0]]
        pr = np.where(pr >= cutoff, pr, 0.0)
        pr = pr / pr.sum()
    cdf = np.cumsum(pr)
    idx = int(np.searchsorted(cdf, u, side="left"))
    return min(idx, V - 1), pr, cdf


def test_brute_force_against_float64_restatement():
    rng = np.random.default_rng(1)
    checked = 0
    for trial in range(600):
        V = int(rng.integers(2, 17))
        lg = rng.normal(0, 2, V).astype(np.float32)
        if trial % 3 == 0:  # force ties
            lg[rng.integers(0, V)] = lg[rng.integers(0, V)]
        T = float(rng.choice([0.5, 0.8, 1.0, 1.7]))
        k = int(rng.integers(0, V + 2))
        p_nuc = float(rng.choice([0.3, 0.6, 0.9, 0.95, 1.0]))
        u = float(rng.random())
        want, pr, cdf = _sample64(lg, T, k, p_nuc, u)
        # skip draws within rounding of a bucket edge or cumulative sums within
        # rounding of top_p: fp32 and fp64 may legitimately land on either side
        srt = np.cumsum(np.sort(_sample64(lg, T, k, 1.0, u)[1])[::-1])
        if np.abs(cdf - u).min() < 1e-5 or (p_nuc < 1 and np.abs(srt - p_nuc).min() < 1e-5):
            continue
        got, gp = O.sample_from_logits(lg, T, k, p_nuc, u, want_probs=True)
        assert np.allclose(gp, pr, atol=2e-6), (lg, T, k, p_nuc)
        assert got == want, (lg, T, k, p_nuc, u)
        checked += 1
    assert checked > 400


# ---- the generate loops (text_gen.cpp:37-91)

def _tiny():
    cfg = synth.Config(synth.ARCH_MODERN, 29, 16, 2, 2, 12)
    W, om = make_pair(cfg, 31, std=0.5)
    return cfg, om


def test_greedy_loop_counts_and_break_rule():
    cfg, om = _tiny()
    assert len(O.generate_greedy(om, [], 5, 1.0)) == 0                 # empty prompt -> nothing (:40)
    toks, sl = O.generate_greedy(om, [1, 2, 3], 4, 1.0, want_logits=True)
    assert len(toks) == 7 and len(sl) == 7                             # every pushed token is stepped (:63)
    # capacity 12: prompt 3 + 9 picks fill it; the 10th pick is pushed, then the loop breaks (:62)
    toks, sl = O.generate_greedy(om, [1, 2, 3], 50, 1.0, want_logits=True)
    assert len(toks) == cfg.max_len + 1 and len(sl) == cfg.max_len
    toks, sl = O.generate_greedy(om, [1, 2, 3], 9, 1.0, want_logits=True)
    assert len(toks) == 12 and len(sl) == 12                           # ends exactly at capacity
    assert len(O.generate_greedy(om, [1, 2, 3], 0, 1.0)) == 3


def test_greedy_loop_is_step_plus_penalised_argmax():
    cfg, om = _tiny()
    for penalty in (1.0, 1.2, 3.0):
        toks = O.generate_greedy(om, [5, 5, 7], 8, penalty)
        s = O.Session(om)
        hist = [5, 5, 7]
        for t in hist:
            lg = s.step(t)
        for _ in range(8):
            adj = lg.astype(np.float32).copy()
            for t in hist[-50:]:
                adj[t] = adj[t] / np.float32(penalty) if adj[t] > 0 else adj[t] * np.float32(penalty)
            nxt = int(np.flatnonzero(adj == adj.max())[0])
            hist.append(nxt)
            lg = s.step(nxt)
        assert toks.tolist() == hist


def test_sample_loop_consumes_one_uniform_per_token():
    cfg, om = _tiny()
    u = synth.uniforms(8, 77)
    toks, sl = O.generate_sample(om, [1, 2, 3], u, 0.8, 8, 1.1, 5, 0.9, want_logits=True)
    assert len(toks) == 11
    hist = [1, 2, 3]
    for i in range(8):
        adj = O.logits_with_penalty(sl[2 + i], hist, 1.1)
        hist.append(O.sample_from_logits(adj, 0.8, 5, 0.9, float(u[i])))
    assert toks.tolist() == hist
    # top_k = 1 makes the draw irrelevant
    a = O.generate_sample(om, [1, 2, 3], synth.uniforms(8, 1), 1.0, 8, 1.0, 1, 1.0)
    b = O.generate_sample(om, [1, 2, 3], synth.uniforms(8, 2), 1.0, 8, 1.0, 1, 1.0)
    assert a.tolist() == b.tolist() == O.generate_greedy(om, [1, 2, 3], 8, 1.0).tolist()


def test_nll_rows_closed_forms():
    """The scoring restatement against what the mathematics fixes."""
    V = 37
    rng = np.random.default_rng(3)
    # uniform logits: -log(1/V) whatever the target and the level
    assert np.allclose(O.nll_rows(np.full((4, V), 2.5), [0, 5, 36, 7]), np.log(V), atol=1e-12)
    # two classes: softplus of the logit difference
    d = rng.normal(size=6) * 3
    x = np.stack([np.zeros(6), d], axis=1)
    assert np.allclose(O.nll_rows(x, np.zeros(6, int)), np.log1p(np.exp(d)), atol=1e-12)
    assert np.allclose(O.nll_rows(x, np.ones(6, int)), np.log1p(np.exp(-d)), atol=1e-12)
    # shift invariance and the definition through probabilities
    x = rng.normal(size=(5, V)) * 4
    t = rng.integers(0, V, 5)
    assert np.allclose(O.nll_rows(x + 100.0, t), O.nll_rows(x, t), atol=1e-9)
    p = np.exp(x) / np.exp(x).sum(axis=1, keepdims=True)
    assert np.allclose(O.nll_rows(x, t), -np.log(p[np.arange(5), t]), atol=1e-12)
    # probabilities sum to one: exp(-nll) over all targets
    assert np.allclose(sum(np.exp(-O.nll_rows(x, np.full(5, j))) for j in range(V)), 1.0, atol=1e-12)
