"""GPU parity: the HIP decode path, called through the C ABI, against the CPU
oracle on the same seeded weights and tokens.  Logits: max|d| <= 1e-4 * max|ref|
per step (fp32 accumulate, different summation order); tokens, cache contents'
indices and counts: exact."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import (TINY_SHAPES, assert_logits_close, check_greedy_stream, check_sampled_stream,
                     lively_std, make_pair, rel_err)

pytestmark = pytest.mark.gpu

TOL = 1e-4


@pytest.fixture(scope="module")
def tiny_models():
    out = {}
    for name, cfg in TINY_SHAPES.items():
        W, om = make_pair(cfg, 11, std=lively_std(cfg), norm_noise=0.1)
        out[name] = (cfg, W, om, G.Model.from_tensors(cfg, W))
    return out


def test_device_is_gfx950():
    info = G.device_info()
    assert info["is_gfx950"], info
    assert info["compute_units"] >= 64


@pytest.mark.parametrize("engine", [G.ENGINE_EAGER, G.ENGINE_GRAPH])
@pytest.mark.parametrize("name", sorted(TINY_SHAPES))
def test_step_logits_and_cache_rows(tiny_models, name, engine):
    cfg, W, om, gm = tiny_models[name]
    gs = G.Session(gm, engine=engine, shuffle_pages=True, page_tokens=4)
    osess = O.Session(om)
    toks = synth.uniform_tokens(cfg.max_len, cfg.vocab, 5)
    for t in toks:
        assert_logits_close(gs.step([t])[0], osess.step(t), TOL, f"{name} step {osess.position}")
    assert gs.position == cfg.max_len == osess.position
    for layer in range(cfg.layers):
        for pos in (0, cfg.max_len // 2, cfg.max_len - 1):
            for kv, row in ((0, osess.k_row(layer, pos)), (1, osess.v_row(layer, pos))):
                got = gs.read_kv(0, layer, kv, pos)
                assert np.abs(got - row).max() <= 2e-5 * max(1.0, float(np.abs(row).max()))


def test_graph_replay_equals_eager_bitwise(tiny_models):
    cfg, W, om, gm = tiny_models["hs64-modern"]
    a, b = G.Session(gm, engine=G.ENGINE_EAGER), G.Session(gm, engine=G.ENGINE_GRAPH)
    for t in synth.uniform_tokens(cfg.max_len, cfg.vocab, 6):
        assert np.array_equal(a.step([t]), b.step([t]))


def test_page_size_and_placement_do_not_change_results(tiny_models):
    cfg, W, om, gm = tiny_models["hs64-gpt2"]
    ref = None
    for page_tokens, shuffle in ((64, False), (4, True), (1, True), (16, False)):
        s = G.Session(gm, page_tokens=page_tokens, shuffle_pages=shuffle)
        out = np.stack([s.step([t])[0] for t in synth.uniform_tokens(cfg.max_len, cfg.vocab, 7)])
        if ref is None:
            ref = out
        assert np.array_equal(ref, out)


@pytest.mark.parametrize("batch", [2, 5, 17, 40, 64])
@pytest.mark.parametrize("name", ["hs64-gpt2", "hs64-modern", "d256-modern", "odd-gpt2", "ref-metal-modern"])
def test_batched_step_equals_per_sequence_oracle(tiny_models, name, batch):
    cfg, W, om, gm = tiny_models[name]
    gs = G.Session(gm, batch=batch, shuffle_pages=True, page_tokens=8)
    toks = synth.uniform_tokens(batch * cfg.max_len, cfg.vocab, 8).reshape(batch, cfg.max_len)
    oss = [O.Session(om) for _ in range(batch)]
    for t in range(cfg.max_len):
        got = gs.step(toks[:, t])
        for b in range(batch):
            assert_logits_close(got[b], oss[b].step(toks[b, t]), TOL, f"{name} B{batch} seq {b} step {t}")


@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("name", ["hs64-gpt2", "hs64-modern", "odd-gpt2", "hs6-modern", "d256-modern"])
def test_attention_split_over_workgroups_merges_to_the_same_logits(tiny_models, name, batch):
    """Long contexts split a (sequence, head) over several workgroups whose partial softmax
    states are merged by the last one to arrive; runs of 16 positions bring that to the tiny
    shapes: up to three partial results per head, the last one ragged."""
    cfg, W, om, gm = tiny_models[name]
    gs = G.Session(gm, batch=batch, flags=G.FLAG_SMALL_ATTENTION_CHUNKS, page_tokens=8, shuffle_pages=True)
    whole = G.Session(gm, batch=batch)
    toks = synth.uniform_tokens(batch * cfg.max_len, cfg.vocab, 12).reshape(batch, cfg.max_len)
    oss = [O.Session(om) for _ in range(batch)]
    for t in range(cfg.max_len):
        got, one = gs.step(toks[:, t]), whole.step(toks[:, t])
        for b in range(batch):
            ref = oss[b].step(toks[b, t])
            assert_logits_close(got[b], ref, TOL, f"{name} B{batch} seq {b} step {t}")
            assert_logits_close(got[b], one[b], 2e-5, f"{name} split vs whole, step {t}")


@pytest.mark.parametrize("arch", [synth.ARCH_GPT2, synth.ARCH_MODERN])
def test_attention_merges_more_than_four_chunks(arch):
    """The merge fetches the partial results of four chunks at a time; up to four go through
    a single round, more through two passes.  A context of 112 in runs of 16 positions walks
    through one to seven chunks per head, ragged and full."""
    cfg = synth.Config(arch, 211, 128, 2, 2, 112)
    W, om = make_pair(cfg, 31, std=lively_std(cfg), norm_noise=0.1)
    gm = G.Model.from_tensors(cfg, W)
    gs = G.Session(gm, batch=2, flags=G.FLAG_SMALL_ATTENTION_CHUNKS, page_tokens=8, shuffle_pages=True)
    whole = G.Session(gm, batch=2)
    toks = synth.uniform_tokens(2 * cfg.max_len, cfg.vocab, 13).reshape(2, cfg.max_len)
    oss = [O.Session(om) for _ in range(2)]
    for t in range(cfg.max_len):
        got, one = gs.step(toks[:, t]), whole.step(toks[:, t])
        for b in range(2):
            assert_logits_close(got[b], oss[b].step(toks[b, t]), TOL, f"seven chunks, arch {arch} seq {b} step {t}")
            assert_logits_close(got[b], one[b], 2e-5, f"seven chunks vs whole, arch {arch} step {t}")


@pytest.mark.parametrize("name", ["hs64-gpt2", "hs64-modern"])
@pytest.mark.parametrize("batch", [1, 3])
def test_prompt_pass_equals_steps(tiny_models, name, batch):
    """Prompts of 8+ tokens run through each layer in one pass; the cache and the
    last logits must be what token-by-token stepping leaves (text_gen.cpp:44-46)."""
    cfg, W, om, gm = tiny_models[name]
    toks = synth.uniform_tokens(batch * 30, cfg.vocab, 9).reshape(batch, 30)
    a = G.Session(gm, batch=batch, shuffle_pages=True, page_tokens=8)
    b = G.Session(gm, batch=batch, flags=G.FLAG_STEPWISE_PROMPT)
    last = a.prefill(toks[:, :19])       # one pass from an empty context
    last = a.prefill(toks[:, 19:])       # and one that continues a context
    ref = b.prefill(toks)
    assert a.position == b.position == 30
    assert_logits_close(last, ref, 2e-5, "prompt pass vs steps")
    for seq in range(batch):
        osess = O.Session(om)
        for t in toks[seq]:
            oref = osess.step(t)
        assert_logits_close(last[seq], oref, TOL, "prompt pass vs oracle")
        for layer in range(cfg.layers):
            for pos in (0, 18, 19, 29):
                for kv, row in ((0, osess.k_row(layer, pos)), (1, osess.v_row(layer, pos))):
                    assert np.abs(a.read_kv(seq, layer, kv, pos) - row).max() <= 2e-5 * max(1.0, float(np.abs(row).max()))
    nxt = synth.uniform_tokens(batch, cfg.vocab, 10)
    assert_logits_close(a.step(nxt), b.step(nxt), 2e-5, "step after prompt pass")
    # short prompts take the token-by-token route
    c = G.Session(gm, batch=batch)
    assert_logits_close(c.prefill(toks[:, :5]), G.Session(gm, batch=batch, flags=G.FLAG_STEPWISE_PROMPT).prefill(toks[:, :5]),
                        1e-6, "short prompt")


@pytest.mark.parametrize("arch", [synth.ARCH_GPT2, synth.ARCH_MODERN])
def test_long_prompt_pass_equals_oracle_steps(arch):
    """Passes of 512 tokens and more run their attention 128 queries per workgroup on the
    32 x 32 x 2 matrix product; shorter ones 64 queries per workgroup.  A 90-token pass,
    then a 650-token pass that continues it (ragged against the 128-query blocks and the
    64-key tiles, over scrambled 8-position pages), then a 530-token pass from an empty
    context over the default pages: last logits and cache rows against the oracle's
    token-by-token steps (inference.cpp:150-258)."""
    cfg = synth.Config(arch, 211, 128, 2, 2, 760)
    W, om = make_pair(cfg, 37, std=lively_std(cfg), norm_noise=0.1)
    gm = G.Model.from_tensors(cfg, W)
    batch = 2
    toks = synth.uniform_tokens(batch * 740, cfg.vocab, 17).reshape(batch, 740)
    a = G.Session(gm, batch=batch, shuffle_pages=True, page_tokens=8)
    a.prefill(toks[:, :90])
    last = a.prefill(toks[:, 90:])
    b = G.Session(gm, batch=batch)
    mid = b.prefill(toks[:, :530])
    assert a.position == 740 and b.position == 530
    for seq in range(batch):
        osess = O.Session(om)
        for i, t in enumerate(toks[seq]):
            oref = osess.step(t)
            if i == 529:
                assert_logits_close(mid[seq], oref, TOL, f"530-token pass, arch {arch} seq {seq}")
        assert_logits_close(last[seq], oref, TOL, f"90 + 650-token passes, arch {arch} seq {seq}")
        for layer in range(cfg.layers):
            for pos in (0, 89, 90, 127, 128, 601, 602, 739):
                for kv, row in ((0, osess.k_row(layer, pos)), (1, osess.v_row(layer, pos))):
                    assert np.abs(a.read_kv(seq, layer, kv, pos) - row).max() <= 2e-5 * max(1.0, float(np.abs(row).max()))


def test_errors_match_the_reference(tiny_models):
    cfg, W, om, gm = tiny_models["ref-sanity-gpt2"]
    s = G.Session(gm)
    with pytest.raises(IndexError, match="InferenceSession: token id out of vocab range"):
        s.step([cfg.vocab])
    with pytest.raises(IndexError, match="InferenceSession: token id out of vocab range"):
        s.step([-1])
    assert s.position == 0
    for _ in range(cfg.max_len):
        s.step([1])
    with pytest.raises(RuntimeError, match="InferenceSession: context exceeds max_len"):
        s.step([1])
    s.reset()
    assert s.position == 0
    s.step([1])
    with pytest.raises(ValueError):
        G.Session(gm, batch=0)
    with pytest.raises(ValueError):
        G.Session(gm, page_tokens=3)


# ---------------------------------------------------------------- generate loops

SAMPLERS = [
    # T, top_k, top_p, penalty
    (0.8, 40, 0.9, 1.1),    # the Llama config's settings
    (1.0, 0, 1.0, 1.2),     # API defaults: no filter (every token survives)
    (0.7, 0, 0.8, 1.0),     # top-p alone (full descending sort)
    (1.3, 5, 1.0, 1.3),     # top-k alone
    (1.0, 1, 1.0, 1.0),     # chat --greedy
]


@pytest.mark.parametrize("flags", [0, G.FLAG_PICK_GLOBAL_SCRATCH])
@pytest.mark.parametrize("name", ["ref-sanity-gpt2", "hs64-modern", "d256-modern"])
@pytest.mark.parametrize("penalty", [1.0, 1.2, 2.5])
def test_generate_greedy_stream(tiny_models, name, penalty, flags):
    cfg, W, om, gm = tiny_models[name]
    prompt = synth.uniform_tokens(5, cfg.vocab, 12)
    prompt[3] = prompt[1]  # a repeated token inside the penalty window
    for max_tokens in (0, 7, cfg.max_len - 5, cfg.max_len + 20):
        ref, rsl = O.generate_greedy(om, prompt, max_tokens, penalty, want_logits=True)
        got, gsl = G.Session(gm, flags=flags).generate(
            prompt, max_tokens, G.sampling(greedy=True, repetition_penalty=penalty), want_logits=True)
        check_greedy_stream(got[0], ref, rsl, len(prompt), f"{name} p{penalty} n{max_tokens}")
        assert got.shape[1] == len(ref) and gsl.shape[0] == len(rsl)  # same number of step() calls
        if np.array_equal(got[0], ref):
            for i in range(len(rsl)):
                assert_logits_close(gsl[i, 0], rsl[i], TOL, f"{name} step {i}")


@pytest.mark.parametrize("flags", [0, G.FLAG_PICK_GLOBAL_SCRATCH])
@pytest.mark.parametrize("name", ["ref-metal-gpt2", "hs64-modern", "d256-modern"])
@pytest.mark.parametrize("opts", SAMPLERS)
def test_generate_sample_stream_under_shared_draws(tiny_models, name, opts, flags):
    cfg, W, om, gm = tiny_models[name]
    T, k, p, pen = opts
    prompt = synth.uniform_tokens(4, cfg.vocab, 13)
    n = cfg.max_len - 4
    u = synth.uniforms(n, 3000)
    ref, rsl = O.generate_sample(om, prompt, u, T, n, pen, k, p, want_logits=True)
    s = G.Session(gm, flags=flags)
    opt = G.sampling(T, k, p, pen)
    got = s.generate(prompt, n, opt, uniforms=u)
    check_sampled_stream(got[0], ref, rsl, len(prompt), u, opts, f"{name} {opts}")
    # the on-device counter-based draws are the same Philox stream
    again = s.generate(prompt, n, opt, seed=3000)
    assert np.array_equal(again, got)
    other = s.generate(prompt, n, opt, seed=3001)
    assert k == 1 or not np.array_equal(other, got)


def test_empty_prompt_generates_nothing(tiny_models):
    cfg, W, om, gm = tiny_models["ref-sanity-gpt2"]
    got = G.Session(gm).generate(np.zeros((1, 0), np.int32), 5, G.sampling(greedy=True))
    assert got.shape == (1, 0)


def test_pick_after_step_matches_generate(tiny_models):
    cfg, W, om, gm = tiny_models["hs64-modern"]
    prompt = synth.uniform_tokens(6, cfg.vocab, 14)
    opt = G.sampling(0.9, 10, 0.95, 1.15)
    u = synth.uniforms(12, 5)
    want = G.Session(gm).generate(prompt, 12, opt, uniforms=u)[0]
    s = G.Session(gm)
    for t in prompt:
        s.step([t])
    out = list(prompt)
    for i in range(12):
        nxt = int(s.pick(opt, uniforms=[u[i]])[0])
        out.append(nxt)
        s.step([nxt])
    assert out == want.tolist()


def test_batched_generate_equals_single_sequence_runs(tiny_models):
    cfg, W, om, gm = tiny_models["hs64-modern"]
    B, plen, n = 6, 5, 20
    prompts = synth.uniform_tokens(B * plen, cfg.vocab, 15).reshape(B, plen)
    u = synth.uniforms(B * n, 16).reshape(B, n)
    for opt in (G.sampling(greedy=True, repetition_penalty=1.2), G.sampling(0.8, 8, 0.9, 1.1)):
        got = G.Session(gm, batch=B).generate(prompts, n, opt, uniforms=u)
        for b in range(B):
            if opt.greedy:
                ref, rsl = O.generate_greedy(om, prompts[b], n, 1.2, want_logits=True)
                check_greedy_stream(got[b], ref, rsl, plen, f"seq {b}")
            else:
                ref, rsl = O.generate_sample(om, prompts[b], u[b], 0.8, n, 1.1, 8, 0.9, want_logits=True)
                check_sampled_stream(got[b], ref, rsl, plen, u[b], (0.8, 8, 0.9, 1.1), f"seq {b}")
