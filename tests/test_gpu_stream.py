"""Streaming decode: TextGen::generate_stream's loop (text_gen.cpp:107-118) hands every
token on as it is sampled.  Here the one-launch engine writes each pick to pinned host
memory while it goes on computing, so the streamed run must give exactly the picks of
the unstreamed one, whatever the callback does, and the two ways of ending early (a
stop token, a request from the callback) must leave the session where a shorter run
would have left it: a later call continues the same stream."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import lively_std

pytestmark = pytest.mark.gpu

CASES = {
    # one launch per run (the persistent engine), both blocks
    "persistent-gpt2": (synth.Config(synth.ARCH_GPT2, 700, 512, 2, 8, 48), 1),
    "persistent-modern": (synth.Config(synth.ARCH_MODERN, 900, 768, 1, 12, 48), 1),
    # one graph replay per step; two sequences
    "graph-modern-b2": (synth.Config(synth.ARCH_MODERN, 301, 128, 2, 2, 40), 2),
    "graph-gpt2": (synth.Config(synth.ARCH_GPT2, 301, 128, 2, 2, 40), 1),
}
OPT = (0.9, 40, 0.95, 1.1)
N = 24


@pytest.fixture(scope="module")
def models():
    out = {}
    for name, (cfg, batch) in CASES.items():
        W = synth.make_weights(cfg, 77, std=lively_std(cfg), norm_noise=0.1)
        out[name] = (cfg, batch, G.Model.from_tensors(cfg, W), W)
    return out


def prompts_of(cfg, batch):
    return np.stack([synth.uniform_tokens(6, cfg.vocab, 40 + b) for b in range(batch)])


def plain_run(gm, cfg, batch, n, seed=5):
    s = G.Session(gm, batch=batch)
    s.prefill(prompts_of(cfg, batch))
    return s.decode(n, G.sampling(*OPT), seed=seed)


@pytest.mark.parametrize("name", sorted(CASES))
def test_engine(models, name):
    cfg, batch, gm, _ = models[name]
    s = G.Session(gm, batch=batch)
    s.generate(prompts_of(cfg, batch), 2, G.sampling(greedy=True))
    assert (s.last_timing()["launches_per_step"] == 1) == name.startswith("persistent")


@pytest.mark.parametrize("name", sorted(CASES))
def test_stream_equals_decode(models, name):
    cfg, batch, gm, _ = models[name]
    ref = plain_run(gm, cfg, batch, N)
    s = G.Session(gm, batch=batch)
    s.prefill(prompts_of(cfg, batch))
    seen = []
    got = s.decode_stream(N, G.sampling(*OPT), lambda ids, i: seen.append((i, list(ids))) and False, seed=5)
    np.testing.assert_array_equal(got, ref)
    assert [i for i, _ in seen] == list(range(N))
    np.testing.assert_array_equal(np.array([ids for _, ids in seen]).T, ref)
    assert s.position == 6 + N


@pytest.mark.parametrize("name", ["persistent-gpt2", "persistent-modern"])
def test_stream_matches_cpu_checker(models, name):
    """The streamed tokens against the CPU restatement under the same uniforms."""
    cfg, batch, gm, W = models[name]
    om = O.Model.from_tensors(cfg, W)
    prompt = prompts_of(cfg, 1)[0]
    u = synth.uniforms(N, 909)
    ref = O.generate_sample(om, prompt, u, OPT[0], N, OPT[3], OPT[1], OPT[2])
    s = G.Session(gm)
    s.prefill(prompt[None, :])
    got = s.decode_stream(N, G.sampling(*OPT), lambda ids, i: False, uniforms=u[None, :])
    np.testing.assert_array_equal(got[0], np.asarray(ref)[len(prompt):])


@pytest.mark.parametrize("name", sorted(CASES))
def test_stop_token_ends_the_run_and_the_next_call_continues(models, name):
    cfg, batch, gm, _ = models[name]
    ref = plain_run(gm, cfg, batch, N)
    # a token every sequence produces, chosen so that the run ends early: the id of
    # sequence 0's eighth pick, unless another sequence never picks it
    stop = int(ref[0, 7])
    last_first = max(int(np.flatnonzero(ref[b] == stop)[0]) if (ref[b] == stop).any() else N - 1
                     for b in range(batch))
    first = last_first + 1  # rounds until every sequence has picked it (or the run is over)
    s = G.Session(gm, batch=batch)
    s.prefill(prompts_of(cfg, batch))
    got = s.decode_stream(N, G.sampling(*OPT), lambda ids, i: False, stop_token=stop, seed=5)
    assert got.shape[1] == first
    np.testing.assert_array_equal(got, ref[:, :first])
    assert s.position == 6 + first
    rest = s.decode(N - first, G.sampling(*OPT), seed=5)
    np.testing.assert_array_equal(rest, ref[:, first:])


@pytest.mark.parametrize("name", sorted(CASES))
def test_callback_can_end_the_run(models, name):
    cfg, batch, gm, _ = models[name]
    ref = plain_run(gm, cfg, batch, N)
    s = G.Session(gm, batch=batch)
    s.prefill(prompts_of(cfg, batch))
    calls = []
    got = s.decode_stream(N, G.sampling(*OPT), lambda ids, i: calls.append(i) or i >= 4, seed=5)
    n = got.shape[1]
    # the request reaches the device a round or two later; every round delivered is complete
    assert 5 <= n <= N
    assert calls == list(range(n))
    if not name.startswith("persistent"):
        assert n == 5
    np.testing.assert_array_equal(got, ref[:, :n])
    assert s.position == 6 + n
    if n < N:
        rest = s.decode_stream(N - n, G.sampling(*OPT), lambda ids, i: False, seed=5)
        np.testing.assert_array_equal(rest, ref[:, n:])


@pytest.mark.parametrize("name", sorted(CASES))
def test_stream_stops_at_capacity(models, name):
    cfg, batch, gm, _ = models[name]
    room = cfg.max_len - 6
    ref = plain_run(gm, cfg, batch, room + 5)
    s = G.Session(gm, batch=batch)
    s.prefill(prompts_of(cfg, batch))
    got = s.decode_stream(room + 5, G.sampling(*OPT), lambda ids, i: False, seed=5)
    # text_gen.cpp:116: the pick made with the context full is delivered, then the loop ends
    assert got.shape[1] == room + 1
    np.testing.assert_array_equal(got, ref)
    assert s.position == cfg.max_len


def test_callback_error_surfaces_after_the_run(models):
    cfg, batch, gm, _ = models["persistent-gpt2"]
    s = G.Session(gm)
    s.prefill(prompts_of(cfg, 1))

    def boom(ids, i):
        if i == 2:
            raise ValueError("from the callback")
        return False

    with pytest.raises(ValueError, match="from the callback"):
        s.decode_stream(N, G.sampling(*OPT), boom, seed=5)
    # the session is still usable and consistent
    assert 6 + 3 <= s.position <= 6 + N
    s.decode(1, G.sampling(*OPT), seed=5)
