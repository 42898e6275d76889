"""Behaviour around the edges of the session API: interleaved sessions on one
model, batches that do not fill the 16-row tiles, prompts shorter and longer
than the one-pass threshold, repeated create/free without leaking device memory."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import assert_logits_close, lively_std, make_pair

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def llama768():
    cfg = synth.Config(synth.ARCH_MODERN, 900, 768, 2, 12, 64)
    W, om = make_pair(cfg, 31, std=0.05, norm_noise=0.1)
    return cfg, W, om, G.Model.from_tensors(cfg, W)


def test_interleaved_sessions_do_not_disturb_each_other(llama768):
    cfg, W, om, gm = llama768
    a = G.Session(gm)                                # persistent engine
    b = G.Session(gm, engine=G.ENGINE_GRAPH)
    c = G.Session(gm, batch=3)                       # batched kernels
    oa, ob = O.Session(om), O.Session(om)
    ta = synth.uniform_tokens(40, cfg.vocab, 1)
    tb = synth.uniform_tokens(40, cfg.vocab, 2)
    for i in range(40):
        ra, rb = oa.step(int(ta[i])), ob.step(int(tb[i]))
        assert_logits_close(a.step([int(ta[i])])[0], ra, 1e-4, f"a step {i}")
        lc = c.step([int(ta[i]), int(tb[i]), int(ta[i])])
        assert_logits_close(b.step([int(tb[i])])[0], rb, 1e-4, f"b step {i}")
        assert_logits_close(lc[0], ra, 1e-4, f"c[0] step {i}")
        assert_logits_close(lc[1], rb, 1e-4, f"c[1] step {i}")
        assert np.array_equal(lc[0], lc[2])


def test_two_host_threads_each_decode_on_a_persistent_session(llama768):
    """Sessions may live on different host threads.  Both run the one-launch engine,
    whose workgroups wait for one another: the library has to keep two such launches
    from sharing the GPU.  Each thread's stream must be the checker's."""
    import threading
    cfg, W, om, gm = llama768
    prompts = [synth.uniform_tokens(9, cfg.vocab, 70 + i) for i in range(2)]
    opt = G.sampling(greedy=True, repetition_penalty=1.0)
    refs = [O.generate_greedy(om, p, 50, 1.0, want_logits=True) for p in prompts]
    got, errs = [None, None], []

    def work(i):
        try:
            s = G.Session(gm, engine=G.ENGINE_PERSISTENT)
            rounds = []
            for _ in range(6):  # many launches per thread, so the two really interleave
                rounds.append(s.generate(prompts[i], 50, opt)[0])
            got[i] = rounds
        except Exception as e:  # noqa: BLE001
            errs.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errs, errs
    from helpers import check_greedy_stream
    for i in range(2):
        for r in got[i]:
            assert np.array_equal(r, got[i][0])
        check_greedy_stream(got[i][0], refs[i][0], refs[i][1], 9, f"thread {i}")


@pytest.mark.parametrize("batch", [7, 19, 33, 130])
def test_batches_that_do_not_fill_a_tile(batch):
    cfg = synth.Config(synth.ARCH_MODERN, 301, 128, 2, 2, 24)
    W, om = make_pair(cfg, 5, std=lively_std(cfg), norm_noise=0.1)
    gm = G.Model.from_tensors(cfg, W)
    s = G.Session(gm, batch=batch)
    toks = np.stack([synth.uniform_tokens(12, cfg.vocab, 40, stream=q) for q in range(batch)])
    last = s.prefill(toks[:, :9])            # one pass (>= 8 tokens)
    more = [s.step(toks[:, 9 + i]) for i in range(3)]
    for q in (0, batch // 2, batch - 1):
        os_ = O.Session(om)
        for t in toks[q, :9]:
            ref = os_.step(int(t))
        assert_logits_close(last[q], ref, 1e-4, f"prompt, sequence {q}")
        for i in range(3):
            assert_logits_close(more[i][q], os_.step(int(toks[q, 9 + i])), 1e-4, f"step {i}, sequence {q}")


@pytest.mark.parametrize("plen", [1, 3, 7, 8, 9, 31])
def test_prompts_around_the_one_pass_threshold(llama768, plen):
    cfg, W, om, gm = llama768
    toks = synth.uniform_tokens(plen + 2, cfg.vocab, 50 + plen)
    os_ = O.Session(om)
    for t in toks[:plen]:
        ref = os_.step(int(t))
    for engine in (G.ENGINE_AUTO, G.ENGINE_GRAPH):
        s = G.Session(gm, engine=engine)
        assert_logits_close(s.prefill(toks[None, :plen])[0], ref, 1e-4, f"prompt of {plen}, engine {engine}")
        assert s.position == plen
        nxt = O.Session(om)
        for t in toks[:plen + 1]:
            r2 = nxt.step(int(t))
        assert_logits_close(s.step([int(toks[plen])])[0], r2, 1e-4, f"step after a prompt of {plen}")


def test_sessions_and_models_give_their_memory_back(llama768):
    import ctypes
    # by soname: the HIP runtime the process already has (the library's, or torch's when
    # torch came first); any other name can bring a second runtime in, which finds no GPU
    hip = ctypes.CDLL("libamdhip64.so.7")

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipDeviceSynchronize() == 0
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    cfg, W, om, gm = llama768
    toks = synth.uniform_tokens(16, cfg.vocab, 3)

    def cycle():
        for engine, batch in ((G.ENGINE_AUTO, 1), (G.ENGINE_GRAPH, 1), (G.ENGINE_AUTO, 5)):
            s = G.Session(gm, batch=batch, engine=engine)
            s.prefill(np.tile(toks[None, :12], (batch, 1)))
            s.decode(3, G.sampling(0.8, 40, 0.9, 1.1), seed=1)
            s.close()
        m2 = G.Model.from_tensors(cfg, W)
        G.Session(m2).step([1])
        del m2

    cycle()
    free0 = free_bytes()
    for _ in range(10):
        cycle()
    free1 = free_bytes()
    assert free0 - free1 < 8 << 20, f"{(free0 - free1) >> 20} MiB not returned after 10 create/free cycles"


def test_prompt_longer_than_one_pass_slice():
    """More prompt rows than one pass takes at a time (32768): the pass runs in slices of
    positions, each attending to the cache rows of the slices before it."""
    cfg = synth.Config(synth.ARCH_MODERN, 301, 128, 1, 2, 1024)
    W = synth.make_weights(cfg, 17, std=lively_std(cfg), norm_noise=0.1)
    om, gm = O.Model.from_tensors(cfg, W), G.Model.from_tensors(cfg, W)
    B, n = 40, 900   # 36000 rows: slices of 819 and 81 positions
    tokens = synth.uniform_tokens(B * (n + 1), cfg.vocab, 18).reshape(B, n + 1)
    ids = np.ascontiguousarray(tokens[:, :-1])
    one_pass = G.Session(gm, batch=B)
    last = one_pass.prefill(ids)
    stepwise = G.Session(gm, batch=B, flags=G.FLAG_STEPWISE_PROMPT)
    want = stepwise.prefill(ids)
    for b in range(B):
        assert_logits_close(last[b], want[b], 2e-5, f"sequence {b}")
    for pos in (0, 818, 819, 899):   # either side of the slice boundary
        for kv in (0, 1):
            assert np.abs(one_pass.read_kv(B - 1, 0, kv, pos) - stepwise.read_kv(B - 1, 0, kv, pos)).max() <= 1e-5
    # one sequence against the CPU oracle, and the scored form of the same pass
    s = O.Session(om)
    for t in ids[7]:
        ref = s.step(int(t))
    assert_logits_close(last[7], ref, 1e-4, "oracle, sequence 7")
    nll = G.Session(gm, batch=B).score(ids, tokens[:, 1:])
    ref_nll = O.score(om, ids[7], tokens[7, 1:])
    assert np.abs(nll[7] - ref_nll).max() <= 2e-4 * max(1.0, np.abs(ref_nll).max())


def test_matrix_core_issue_probe():
    """gh_device_mfma_issue: a dependent chain of v_mfma_f32_32x32x2_f32 runs at one product per
    64 cycles, and the probe refuses modes and slot sizes it has no kernel for."""
    prod, slot, mhz = G.mfma_issue(1, 8)
    assert 60.0 < prod < 70.0 and slot == 0.0 and 1000.0 < mhz < 3000.0
    prod, slot, mhz = G.mfma_issue(2, 8)
    assert prod == 0.0 and 20.0 < slot < 60.0
    for mode, per in ((0, 8), (5, 8), (7, 8), (1, 9)):
        with pytest.raises(Exception):
            G.mfma_issue(mode, per)
