"""Shared test helpers: seeded models on both sides, comparison rules."""
from __future__ import annotations

import numpy as np

import oracle_lib as O
from gradhip import synth

# The reference's own parity-test shapes (tests/integration/sanity_tests.cpp:296-301,
# tests/integration/metal_parity.cpp:345-379) plus a head-size-64 shape.
TINY_SHAPES = {
    "ref-sanity-gpt2": synth.Config(synth.ARCH_GPT2, 23, 32, 2, 4, 16),
    "ref-sanity-modern": synth.Config(synth.ARCH_MODERN, 23, 32, 2, 4, 16),
    "ref-metal-gpt2": synth.Config(synth.ARCH_GPT2, 97, 64, 2, 4, 16),
    "ref-metal-modern": synth.Config(synth.ARCH_MODERN, 97, 64, 2, 4, 16),
    "hs64-gpt2": synth.Config(synth.ARCH_GPT2, 301, 128, 2, 2, 40),
    "hs64-modern": synth.Config(synth.ARCH_MODERN, 301, 128, 2, 2, 40),
    "odd-gpt2": synth.Config(synth.ARCH_GPT2, 37, 21, 2, 3, 12),      # d % 4 != 0, head size 7
    "hs6-modern": synth.Config(synth.ARCH_MODERN, 50, 24, 2, 4, 20),  # head size 6 (any-size path)
    "d256-modern": synth.Config(synth.ARCH_MODERN, 1000, 256, 2, 4, 48),  # vector path, K = 256
}
REF_SEQUENCE = [3, 11, 7, 0, 19, 5]  # sanity_tests.cpp:301


def rel_err(a, b):
    """max |a-b| / max |b|: the per-step logits rule (1e-4 relative, fp32 accumulate)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


# Worst observed values of the two logits rules per label, and where the per-element
# one was seen, for the record a GPU run prints at its end (tests/conftest.py).
WORST = {}


def assert_logits_close(got, ref, tol=1e-4, what="", abs_term=None):
    """The per-step logits rule: max|d| <= tol * max|ref| for the step, and per
    element |d_i| <= tol * max(|got_i|, |ref_i|) + abs_term (summation-order noise
    is absolute, so an element near zero cannot be held to its own magnitude).
    abs_term defaults to 5e-6 of the step's largest logit (the named configurations
    stay below 1.5e-6 of it, the tiny shapes with livelier weights reach 3.2e-6).  (An absolute 1e-6 is
    below the rounding of two correct fp32 implementations here: the 22M GPT-2
    configuration has logits beyond 1.4, and its first step already differs from
    the checker by 1.4e-6 on an element near zero while its max-norm error is 1e-6
    relative.)
    grad.cpp's own parity test allows 1e-3 + 1e-3 * (|a| + |b|)
    (tests/integration/sanity_tests.cpp:322)."""
    e = rel_err(got, ref)
    a, b = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    if abs_term is None:
        abs_term = 5e-6 * float(np.abs(b).max())
    share = np.abs(a - b) / (tol * np.maximum(np.abs(a), np.abs(b)) + abs_term)
    per = float(share.max())
    label = what.split(" step ")[0].split(" decode ")[0] or "unnamed"
    w = WORST.setdefault(label, [0.0, 0.0, ""])
    w[0] = max(w[0], e / tol)
    if per > w[1]:
        i = int(share.reshape(-1).argmax())
        big = max(float(np.abs(b).max()), 1e-30)
        w[1] = per
        w[2] = (f"{what or 'unnamed'}, element {i}: |ref| = {abs(b.reshape(-1)[i]) / big:.4f} of the step's largest, "
                f"|d| = {abs(a.reshape(-1)[i] - b.reshape(-1)[i]) / big:.2e} of it")
    assert e <= tol, f"{what}: max|d|/max|ref| = {e:.3e} > {tol}"
    assert per <= 1.0, f"{what}: per-element rule exceeded ({per:.3f} of the allowance)"


def top2_margin(logits):
    s = np.sort(np.asarray(logits, dtype=np.float64))
    return float(s[-1] - s[-2])


def lively_std(cfg):
    """A weight scale for the tiny test shapes that makes attention and the
    activations clearly non-linear (pre-activations of order 1) without driving
    the network into a regime that amplifies fp32 rounding chaotically."""
    return min(0.2, 1.13 / float(np.sqrt(cfg.d_model)))


def make_pair(cfg, seed, std=0.02, norm_noise=0.0):
    """(weights, oracle model) for a config."""
    W = synth.make_weights(cfg, seed, std=std, norm_noise=norm_noise)
    return W, O.Model.from_tensors(cfg, W)


def check_greedy_stream(got, ref, ref_step_logits, n_prompt, what=""):
    """Token streams must be identical; a divergence is tolerated only where the
    oracle's own top-2 margin is below the fp32 summation-order noise (a genuine
    near-tie between two correct implementations), and is reported."""
    got, ref = np.asarray(got), np.asarray(ref)
    n = min(len(got), len(ref))
    diff = np.flatnonzero(got[:n] != ref[:n])
    if len(got) == len(ref) and len(diff) == 0:
        return None
    assert len(diff) > 0, f"{what}: lengths differ ({len(got)} vs {len(ref)}) with equal prefixes"
    i = int(diff[0])
    assert i >= n_prompt, f"{what}: prompt echoed wrongly at {i}"
    lg = ref_step_logits[i - 1]                  # the logits token i was picked from
    margin = top2_margin(lg)
    noise = 4e-6 * float(np.abs(lg).max())
    assert margin <= noise, (f"{what}: streams diverge at token {i} ({got[i]} vs {ref[i]}) with a "
                             f"top-2 margin of {margin:.3e} (noise floor {noise:.1e})")
    return i


def check_sampled_stream(got, ref, ref_step_logits, n_prompt, uniforms, opts, what=""):
    """Same draws must give the same stream, except where the draw sits within
    rounding of a CDF bucket edge of the oracle's own distribution."""
    got, ref = np.asarray(got), np.asarray(ref)
    n = min(len(got), len(ref))
    diff = np.flatnonzero(got[:n] != ref[:n])
    if len(got) == len(ref) and len(diff) == 0:
        return None
    assert len(diff) > 0
    i = int(diff[0])
    assert i >= n_prompt
    T, k, p, pen = opts
    adj = O.logits_with_penalty(ref_step_logits[i - 1], ref[:i], pen)
    _, probs = O.sample_from_logits(adj, T, k, p, 0.5, want_probs=True)
    cdf = np.cumsum(probs.astype(np.float64))
    u = float(uniforms[i - n_prompt])
    assert np.abs(cdf - u).min() < 2e-5, (f"{what}: sampled streams diverge at token {i} with the "
                                          f"draw {u} not near a bucket edge")
    return i
