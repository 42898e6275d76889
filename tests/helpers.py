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


def assert_logits_close(got, ref, tol=1e-4, what=""):
    e = rel_err(got, ref)
    assert e <= tol, f"{what}: max|d|/max|ref| = {e:.3e} > {tol}"
    # element rule: |d| <= tol * max(|a|,|b|) + 1e-6
    a, b = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    bad = np.abs(a - b) > tol * np.maximum(np.abs(a), np.abs(b)) + 1e-6 + tol * np.abs(b).max() * 0.01
    assert not bad.any(), f"{what}: {int(bad.sum())} elements outside the per-element rule"


def top2_margin(logits):
    s = np.sort(np.asarray(logits, dtype=np.float64))
    return float(s[-1] - s[-2])


def make_pair(cfg, seed, std=0.02, norm_noise=0.0):
    """(weights, oracle model) for a config."""
    W = synth.make_weights(cfg, seed, std=std, norm_noise=norm_noise)
    return W, O.Model.from_tensors(cfg, W)
