"""Vocabularies beyond the benchmark's 16000: the sizes real tokenizers have
(32000, 50257) and one past every fast path.  The sampler changes shape with the
vocabulary - more elements per thread, then a working row that no longer fits in
LDS and lives in global memory, then passes that re-read the row - and every
shape has to give the reference's streams (text_gen.cpp:14-209)."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import check_greedy_stream, check_sampled_stream, lively_std

pytestmark = pytest.mark.gpu

CASES = {
    # more than 32 elements per sampler thread, row still in LDS
    "v32000": synth.Config(synth.ARCH_MODERN, 32000, 64, 1, 2, 40),
    # row in global memory
    "v50257": synth.Config(synth.ARCH_GPT2, 50257, 64, 1, 2, 40),
    # more than 64 elements per sampler thread: the passes re-read the row
    "v70001": synth.Config(synth.ARCH_MODERN, 70001, 64, 1, 2, 40),
    # the one-launch engine with the row in LDS (512 sampler threads, 63 elements each)
    "persistent-v32000": synth.Config(synth.ARCH_GPT2, 32000, 512, 1, 8, 40),
    # the one-launch engine with the row in global memory
    "persistent-v50257": synth.Config(synth.ARCH_MODERN, 50257, 768, 1, 12, 40),
}
SAMPLERS = [
    (0.8, 40, 0.9, 1.1),
    (1.0, 0, 1.0, 1.2),
    (0.7, 0, 0.8, 1.0),
    (1.2, 64, 1.0, 1.3),
    (1.0, 300, 0.95, 1.0),
]


@pytest.fixture(scope="module")
def models():
    out = {}
    for name, cfg in CASES.items():
        W = synth.make_weights(cfg, 91, std=lively_std(cfg), norm_noise=0.1)
        out[name] = (cfg, O.Model.from_tensors(cfg, W), G.Model.from_tensors(cfg, W))
    return out


@pytest.mark.parametrize("name", sorted(CASES))
def test_engine_choice(models, name):
    cfg, om, gm = models[name]
    s = G.Session(gm)
    s.generate(synth.uniform_tokens(3, cfg.vocab, 20), 2, G.sampling(greedy=True))
    assert (s.last_timing()["launches_per_step"] == 1) == name.startswith("persistent")


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("penalty", [1.0, 1.3])
def test_greedy_stream(models, name, penalty):
    cfg, om, gm = models[name]
    prompt = synth.uniform_tokens(5, cfg.vocab, 21)
    prompt[3] = prompt[0]
    n = 20
    ref, rsl = O.generate_greedy(om, prompt, n, penalty, want_logits=True)
    got = G.Session(gm).generate(prompt, n, G.sampling(greedy=True, repetition_penalty=penalty))
    check_greedy_stream(got[0], ref, rsl, len(prompt), f"{name} p{penalty}")


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("opts", SAMPLERS)
def test_sampled_stream_under_shared_draws(models, name, opts):
    cfg, om, gm = models[name]
    T, k, p, pen = opts
    prompt = synth.uniform_tokens(4, cfg.vocab, 22)
    n = 24
    u = synth.uniforms(n, 4100)
    u[5] = 0.0  # a zero draw picks index 0 (text_gen.cpp:202-208)
    ref, rsl = O.generate_sample(om, prompt, u, T, n, pen, k, p, want_logits=True)
    got = G.Session(gm).generate(prompt, n, G.sampling(T, k, p, pen), uniforms=u)
    check_sampled_stream(got[0], ref, rsl, len(prompt), u, opts, f"{name} {opts}")


@pytest.mark.parametrize("name", ["v50257", "persistent-v50257"])
def test_host_loop_matches_generate(models, name):
    """step() + pick() from the host against the on-device loop, with the row in global memory."""
    cfg, om, gm = models[name]
    prompt = synth.uniform_tokens(6, cfg.vocab, 23)
    opt = G.sampling(0.9, 10, 0.95, 1.15)
    u = synth.uniforms(10, 6)
    want = G.Session(gm).generate(prompt, 10, opt, uniforms=u)[0]
    s = G.Session(gm)
    for t in prompt:
        s.step([t])
    out = list(prompt)
    for i in range(10):
        nxt = int(s.pick(opt, uniforms=[u[i]])[0])
        out.append(nxt)
        s.step([nxt])
    assert out == list(want)
