"""The sampler where it is easiest to get wrong: exact ties.  With tied embeddings,
duplicated rows of E give bit-identical logits for the duplicated tokens in any
implementation, so whole groups of tokens tie at the top-k threshold (they must
all survive, text_gen.cpp:150-154), tie in the descending top-p order and tie for
the arg-max (lowest index wins, text_gen.cpp:52-60).  The survivor counts are
chosen to cross the limits of the GPU sampler's fast path (64 survivors, 512
candidates), so its fallbacks run too."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import check_greedy_stream, check_sampled_stream, lively_std

pytestmark = pytest.mark.gpu

CASES = {
    # name: (config, distinct embedding rows)
    "small": (synth.Config(synth.ARCH_MODERN, 600, 128, 2, 2, 40), 37),       # groups of ~16 tokens
    "wide-groups": (synth.Config(synth.ARCH_GPT2, 1500, 128, 2, 2, 40), 3),   # groups of 500 tokens
    "persistent": (synth.Config(synth.ARCH_MODERN, 1200, 768, 2, 12, 48), 50),  # groups of 24, one-launch engine
    # every workgroup of the one-launch engine has rows of the logits: top-k picks are made from four
    # candidates per workgroup, and ties at the cut hand the pick back to the whole row
    "persistent-wide": (synth.Config(synth.ARCH_MODERN, 4096, 768, 1, 12, 40), 500),
}
SAMPLERS = [
    (1.0, 40, 0.9, 1.0),   # the threshold group straddles k = 40
    (1.0, 5, 1.0, 1.2),    # k inside the first group; penalty breaks some ties
    (0.9, 60, 0.8, 1.1),   # ~64 survivors
    (1.1, 64, 0.95, 1.0),  # more than 64 survivors
    (0.8, 0, 0.7, 1.3),    # top-p alone over tied probabilities
]


def tied_model(cfg, distinct, seed):
    W = synth.make_weights(cfg, seed, std=lively_std(cfg), norm_noise=0.1)
    E = W[0]
    assert E.shape == (cfg.vocab, cfg.d_model)
    E[:] = E[np.arange(cfg.vocab) % distinct]
    return W, O.Model.from_tensors(cfg, W), G.Model.from_tensors(cfg, W)


@pytest.fixture(scope="module")
def models():
    return {name: (cfg,) + tied_model(cfg, distinct, 77) for name, (cfg, distinct) in CASES.items()}


@pytest.mark.parametrize("name", sorted(CASES))
def test_tied_logits_are_bitwise_tied_on_the_gpu(models, name):
    cfg, W, om, gm = models[name]
    distinct = CASES[name][1]
    s = G.Session(gm)
    logits = s.step([3])[0]
    for r in range(min(distinct, 5)):
        group = logits[r::distinct]
        assert np.all(group == group[0])


@pytest.mark.parametrize("flags", [0, G.FLAG_PICK_GLOBAL_SCRATCH])
@pytest.mark.parametrize("opts", SAMPLERS)
@pytest.mark.parametrize("name", sorted(CASES))
def test_sampled_streams_with_ties(models, name, opts, flags):
    cfg, W, om, gm = models[name]
    T, k, p, pen = opts
    prompt = synth.uniform_tokens(5, cfg.vocab, 31)
    n = cfg.max_len - 5
    u = synth.uniforms(n, 4100)
    ref, rsl = O.generate_sample(om, prompt, u, T, n, pen, k, p, want_logits=True)
    s = G.Session(gm, flags=flags)
    got = s.generate(prompt, n, G.sampling(T, k, p, pen), uniforms=u)
    check_sampled_stream(got[0], ref, rsl, len(prompt), u, opts, f"{name} {opts} flags={flags}")


@pytest.mark.parametrize("name", sorted(CASES))
def test_greedy_picks_the_lowest_tied_index(models, name):
    cfg, W, om, gm = models[name]
    distinct = CASES[name][1]
    prompt = synth.uniform_tokens(5, cfg.vocab, 32)
    n = cfg.max_len - 5
    ref, rsl = O.generate_greedy(om, prompt, n, 1.0, want_logits=True)
    got, _ = G.Session(gm).generate(prompt, n, G.sampling(greedy=True, repetition_penalty=1.0), want_logits=True)
    check_greedy_stream(got[0], ref, rsl, len(prompt), name)
    assert np.all(np.asarray(ref[len(prompt):]) < distinct)  # always the first copy of the winning row


@pytest.mark.parametrize("engine", [G.ENGINE_GRAPH, G.ENGINE_EAGER])
@pytest.mark.parametrize("batch", [16, 32, 64])
def test_batched_greedy_picks_the_lowest_tied_index(batch, engine):
    """Batched greedy decoding without a penalty takes its pick from what the logits launch
    leaves per run of 16 columns (the few-rows kernel at 16 and 32 sequences, the tiled one
    at 64) and embeds it in the same launch: ties across runs, tiles and workgroups must
    still go to the lowest index, for every sequence."""
    cfg = synth.Config(synth.ARCH_GPT2, 9000, 512, 1, 8, 24)
    distinct = 7
    W, om, gm = tied_model(cfg, distinct, 78)
    prompts = np.stack([synth.uniform_tokens(4, cfg.vocab, 33, stream=b) for b in range(batch)])
    n = cfg.max_len - 4 + 3  # runs into the capacity rule: the last pick has no step behind it
    s = G.Session(gm, batch=batch, engine=engine)
    got = s.generate(prompts, n, G.sampling(greedy=True, repetition_penalty=1.0))
    for b in range(0, batch, max(1, batch // 8)):
        ref, rsl = O.generate_greedy(om, prompts[b], n, 1.0, want_logits=True)
        check_greedy_stream(got[b], ref, rsl, 4, f"batch {batch} sequence {b}")
        assert np.all(np.asarray(ref[4:]) < distinct)
    # the same through decode calls that continue one context
    s.reset()
    s.prefill(prompts)
    a = s.decode(5, G.sampling(greedy=True, repetition_penalty=1.0))
    b2 = s.decode(n - 5, G.sampling(greedy=True, repetition_penalty=1.0))
    np.testing.assert_array_equal(np.concatenate([prompts, a, b2], axis=1), got)
