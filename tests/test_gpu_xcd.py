"""The XCD-sharded persistent kernel (a layer split over the eight XCDs, weights
streamed through LDS) against the CPU checker and against the all-to-all persistent
kernel: steps, the generate loops with every sampler setting, the streaming entry
point with both ways of ending early, attention spread over every workgroup of an
XCD, and a context long enough for several passes per slice."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import assert_logits_close, check_greedy_stream, check_sampled_stream, make_pair

pytestmark = pytest.mark.gpu

CFG = synth.Config(synth.ARCH_MODERN, 1200, 768, 2, 12, 96)
XCD = G.FLAG_XCD_PERSISTENT


@pytest.fixture(scope="module")
def model():
    W, om = make_pair(CFG, 21, std=0.05, norm_noise=0.1)
    return W, om, G.Model.from_tensors(CFG, W)


def xcd_session(gm, **kw):
    flags = kw.pop("flags", 0) | XCD
    return G.Session(gm, engine=G.ENGINE_PERSISTENT, flags=flags, **kw)


def test_steps_match_the_checker_and_the_other_kernel(model):
    W, om, gm = model
    x = xcd_session(gm)
    shuffled = xcd_session(gm, shuffle_pages=True, page_tokens=8)
    wide = xcd_session(gm, flags=G.FLAG_SMALL_ATTENTION_CHUNKS)  # every workgroup of an XCD takes a slice
    classic = G.Session(gm, engine=G.ENGINE_PERSISTENT, flags=G.FLAG_CLASSIC_PERSISTENT)
    osess = O.Session(om)
    for t in synth.uniform_tokens(CFG.max_len, CFG.vocab, 5):
        ref = osess.step(t)
        a = x.step([t])[0]
        assert_logits_close(a, ref, 1e-4, f"xcd llama-d768 step {osess.position}")
        assert np.array_equal(a, shuffled.step([t])[0])  # page placement does not matter
        assert_logits_close(wide.step([t])[0], ref, 1e-4, f"xcd-all-slices llama-d768 step {osess.position}")
        assert_logits_close(classic.step([t])[0], a, 2e-5)  # two kernels, same numbers up to sum order
    with pytest.raises(RuntimeError, match="InferenceSession: context exceeds max_len"):
        x.step([1])
    for layer in range(CFG.layers):
        for pos in (0, 37, CFG.max_len - 1):
            assert np.abs(shuffled.read_kv(0, layer, 0, pos) - osess.k_row(layer, pos)).max() < 2e-5
            assert np.abs(shuffled.read_kv(0, layer, 1, pos) - osess.v_row(layer, pos)).max() < 2e-5


def test_generate_loops(model):
    W, om, gm = model
    prompt = synth.uniform_tokens(7, CFG.vocab, 6)
    prompt[4] = prompt[2]
    n = CFG.max_len - 7 + 5  # runs into the capacity rule
    u = synth.uniforms(n, 9)
    s = xcd_session(gm)
    for penalty in (1.0, 1.2):
        ref, rsl = O.generate_greedy(om, prompt, n, penalty, want_logits=True)
        got, gsl = s.generate(prompt, n, G.sampling(greedy=True, repetition_penalty=penalty), want_logits=True)
        check_greedy_stream(got[0], ref, rsl, 7, f"xcd greedy {penalty}")
        assert got.shape[1] == len(ref) == CFG.max_len + 1 and len(gsl) == len(rsl) == CFG.max_len
        for i in (0, len(rsl) // 2, len(rsl) - 1):
            assert_logits_close(gsl[i, 0], rsl[i], 1e-4, f"xcd generate step {i}")
    for opts in ((0.8, 40, 0.9, 1.1), (1.0, 0, 1.0, 1.2), (0.7, 0, 0.8, 1.0), (1.3, 5, 1.0, 1.3)):
        T, k, p, pen = opts
        ref, rsl = O.generate_sample(om, prompt, u, T, n, pen, k, p, want_logits=True)
        got = s.generate(prompt, n, G.sampling(T, k, p, pen), uniforms=u)
        check_sampled_stream(got[0], ref, rsl, 7, u, opts, f"xcd {opts}")
        assert np.array_equal(s.generate(prompt, n, G.sampling(T, k, p, pen), seed=9), got)


@pytest.mark.parametrize("flags", [0, G.FLAG_PICK_GLOBAL_SCRATCH])
def test_prefill_then_decode_continues_the_context(model, flags):
    """Prompt passes by the batched kernels, then runs of the XCD kernel, with the
    sampler's row in LDS and in global memory."""
    W, om, gm = model
    prompt = synth.uniform_tokens(20, CFG.vocab, 7)
    opt = G.sampling(0.9, 10, 0.95, 1.15)
    u = synth.uniforms(30, 8)
    whole = G.Session(gm, engine=G.ENGINE_PERSISTENT, flags=G.FLAG_CLASSIC_PERSISTENT).generate(prompt, 30, opt, uniforms=u)[0]
    s = xcd_session(gm, flags=flags)
    s.prefill(prompt[:11])
    s.prefill(prompt[11:])
    a = s.decode(12, opt, uniforms=u[:12])[0]
    b = s.decode(18, opt, uniforms=u[12:])[0]
    assert np.concatenate([prompt, a, b]).tolist() == whole.tolist()


def test_streaming_and_both_ways_of_ending_early(model):
    W, om, gm = model
    opt = G.sampling(0.9, 40, 0.95, 1.1)
    prompt = synth.uniform_tokens(6, CFG.vocab, 40)[None, :]
    N = 24

    def fresh():
        s = xcd_session(gm)
        s.prefill(prompt)
        return s

    ref = fresh().decode(N, opt, seed=5)
    seen = []
    s = fresh()
    got = s.decode_stream(N, opt, lambda ids, i: seen.append(int(ids[0])) and False, seed=5)
    np.testing.assert_array_equal(got, ref)
    assert seen == ref[0].tolist() and s.position == 6 + N
    # a stop token ends the run after the step that follows it; a later call continues the stream
    stop = int(ref[0, 7])
    first = int(np.flatnonzero(ref[0] == stop)[0]) + 1
    s = fresh()
    got = s.decode_stream(N, opt, lambda ids, i: False, stop_token=stop, seed=5)
    np.testing.assert_array_equal(got, ref[:, :first])
    assert s.position == 6 + first
    np.testing.assert_array_equal(s.decode(N - first, opt, seed=5), ref[:, first:])
    # a request from the callback
    s = fresh()
    got = s.decode_stream(N, opt, lambda ids, i: i >= 4, seed=5)
    n = got.shape[1]
    assert 5 <= n <= N and s.position == 6 + n
    np.testing.assert_array_equal(got, ref[:, :n])
    if n < N:
        np.testing.assert_array_equal(s.decode(N - n, opt, seed=5), ref[:, n:])


def test_long_context_on_both_kernels():
    """Beyond 256 positions every workgroup of an XCD takes a slice of the attention, and
    beyond 32 positions per slice a slice is walked in several passes.  A session
    without a flag stays on the all-to-all kernel at every position (which shares a
    head's context among workgroups from 512 positions on); the two kernels must agree
    with the checker and with each other along one long context."""
    cfg = synth.Config(synth.ARCH_MODERN, 500, 768, 1, 12, 1300)
    W, om = make_pair(cfg, 23, std=0.05, norm_noise=0.1)
    gm = G.Model.from_tensors(cfg, W)
    forced = G.Session(gm, engine=G.ENGINE_PERSISTENT, flags=XCD)
    auto = G.Session(gm, engine=G.ENGINE_PERSISTENT)
    osess = O.Session(om)
    toks = synth.uniform_tokens(cfg.max_len, cfg.vocab, 8)
    for t in toks[:1000]:
        ref = osess.step(int(t))
    assert_logits_close(forced.prefill(toks[None, :1000])[0], ref, 1e-4, "after a 1000-token prompt")
    auto.prefill(toks[None, :1000])
    for i, t in enumerate(toks[1000:]):
        ref = osess.step(int(t))
        a = forced.step([int(t)])[0]
        b = auto.step([int(t)])[0]  # the all-to-all kernel, a head's context in four to six shares
        if i % 20 == 0 or i >= len(toks) - 1003:
            assert_logits_close(a, ref, 1e-4, f"xcd position {1000 + i}")
            assert_logits_close(b, ref, 1e-4, f"auto position {1000 + i}")
        assert_logits_close(b, a, 2e-5)  # two kernels: same up to sum order
    # one launch that runs through the rest of a long context
    s = G.Session(gm, engine=G.ENGINE_PERSISTENT, flags=XCD)
    s.prefill(toks[None, :1100])
    got = s.decode(150, G.sampling(greedy=True, repetition_penalty=1.0))[0]
    ref, rsl = O.generate_greedy(om, toks[:1100], 150, 1.0, want_logits=True)
    check_greedy_stream(np.concatenate([toks[:1100], got]), ref, rsl, 1100, "xcd long greedy run")


def test_flags_exclude_each_other(model):
    W, om, gm = model
    with pytest.raises(ValueError, match="exclude each other"):
        G.Session(gm, engine=G.ENGINE_PERSISTENT, flags=G.FLAG_XCD_PERSISTENT | G.FLAG_CLASSIC_PERSISTENT)
