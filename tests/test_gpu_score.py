"""gh_session_score: the per-position negative log-likelihood `grad eval` averages
(training/trainer.cpp:319-340), computed for all positions in one pass over the weights,
against the CPU restatement (step() logits -> float64 log-softmax)."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import assert_logits_close, lively_std

pytestmark = pytest.mark.gpu

CASES = {
    # name: (config, batch, window length)
    "tiny-gpt2-stepwise": (synth.Config(synth.ARCH_GPT2, 97, 64, 2, 4, 40), 2, 24),     # head size 16: token by token
    "hs64-modern": (synth.Config(synth.ARCH_MODERN, 301, 128, 2, 2, 64), 3, 40),         # one pass, small tiles
    "hs64-gpt2": (synth.Config(synth.ARCH_GPT2, 301, 128, 2, 2, 64), 3, 40),
    "big-tiles": (synth.Config(synth.ARCH_MODERN, 1000, 256, 2, 4, 192), 4, 160),        # 640 rows: 128 x 128 tiles
    "blocks-of-rows": (synth.Config(synth.ARCH_MODERN, 70001, 128, 1, 2, 96), 12, 90),   # logits in several blocks
    "persistent-short": (synth.Config(synth.ARCH_GPT2, 500, 512, 1, 8, 32), 1, 5),       # shorter than one pass takes
    "persistent-pass": (synth.Config(synth.ARCH_GPT2, 500, 512, 1, 8, 32), 1, 20),
}


@pytest.fixture(scope="module")
def models():
    out = {}
    for name, (cfg, B, n) in CASES.items():
        W = synth.make_weights(cfg, 55, std=lively_std(cfg), norm_noise=0.1)
        out[name] = (cfg, B, n, O.Model.from_tensors(cfg, W), G.Model.from_tensors(cfg, W))
    return out


@pytest.mark.parametrize("name", sorted(CASES))
def test_score_matches_the_oracle(models, name):
    cfg, B, n, om, gm = models[name]
    tokens = synth.uniform_tokens(B * (n + 1), cfg.vocab, 61).reshape(B, n + 1)
    ids, targets = tokens[:, :-1], tokens[:, 1:]   # next-token targets, as the data loader pairs them
    s = G.Session(gm, batch=B)
    got = s.score(ids, targets)
    assert got.shape == (B, n) and s.position == n
    check = range(B) if name != "blocks-of-rows" else (0, B - 1)   # the CPU side is slow at this vocabulary
    for b in check:
        ref = O.score(om, ids[b], targets[b])
        # NLL = logsumexp - logit: both terms carry the logits' error
        scale = max(1.0, float(np.abs(ref).max()))
        assert np.abs(got[b] - ref).max() <= 2e-4 * scale, (name, b, np.abs(got[b] - ref).max())
    # the mean, as mean_loss reports it
    if name != "blocks-of-rows":
        ref_mean = np.mean([O.score(om, ids[b], targets[b]).mean() for b in range(B)])
        assert abs(got.mean(dtype=np.float64) - ref_mean) <= 1e-4 * max(1.0, ref_mean)


def test_score_leaves_the_cache_of_a_prefill(models):
    cfg, B, n, om, gm = models["hs64-modern"]
    tokens = synth.uniform_tokens(B * (n + 1), cfg.vocab, 62).reshape(B, n + 1)
    a, b = G.Session(gm, batch=B), G.Session(gm, batch=B)
    a.score(tokens[:, :-1], tokens[:, 1:])
    b.prefill(tokens[:, :-1])
    nxt = tokens[:, -1]
    assert_logits_close(a.step(nxt), b.step(nxt), 1e-6)


def test_score_in_two_windows_continues_the_context(models):
    cfg, B, n, om, gm = models["hs64-gpt2"]
    tokens = synth.uniform_tokens(B * (n + 1), cfg.vocab, 63).reshape(B, n + 1)
    whole = G.Session(gm, batch=B).score(tokens[:, :-1], tokens[:, 1:])
    s = G.Session(gm, batch=B)
    first = s.score(tokens[:, :16], tokens[:, 1:17])
    second = s.score(tokens[:, 16:n], tokens[:, 17:n + 1])
    assert np.abs(np.concatenate([first, second], axis=1) - whole).max() <= 1e-5 * max(1.0, np.abs(whole).max())


def test_score_errors(models):
    cfg, B, n, om, gm = models["hs64-modern"]
    s = G.Session(gm, batch=B)
    ok = np.zeros((B, 8), np.int32)
    bad = ok.copy()
    bad[1, 3] = cfg.vocab
    with pytest.raises(IndexError, match="token id out of vocab range"):
        s.score(bad, ok)
    with pytest.raises(IndexError, match="token id out of vocab range"):
        s.score(ok, bad)
    with pytest.raises(RuntimeError, match="context exceeds max_len"):
        s.score(np.zeros((B, cfg.max_len + 1), np.int32), np.zeros((B, cfg.max_len + 1), np.int32))
    assert s.position == 0
