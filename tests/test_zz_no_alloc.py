"""gh_pick_noalloc, the entry point that allocates nothing: its picks must be those of
gh_session_pick, and of the CPU checker, on the same logits, history, options and draws, on two calls in a row,
the second with a smaller input (the shared working rows keep the first call's
contents).  Device memory for the caller's side comes from torch."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth

pytestmark = pytest.mark.gpu


def _torch_on_the_loaded_runtime():
    """torch, sharing the HIP runtime the library has brought up.  torch ships a copy of
    the runtime and asks the loader for it as "libamdhip64.so"; a second runtime in one
    process finds no GPU.  Loading that name first makes the loader hand torch the file
    that is already mapped (the library links the same file under its soname)."""
    import ctypes
    G.device_info()  # the documented set-up call; loads the library and its runtime
    ctypes.CDLL("libamdhip64.so")
    return pytest.importorskip("torch")

OPTIONS = [
    dict(greedy=True, repetition_penalty=1.3),
    dict(temperature=0.8, top_k=40, top_p=0.9, repetition_penalty=1.1),
    dict(temperature=1.3, top_k=0, top_p=0.7, repetition_penalty=1.0),
    dict(temperature=1.0, top_k=200, top_p=1.0, repetition_penalty=1.2),
]


def _case(torch, cfg, seed, batch, plen):
    """Logits and history of `batch` sequences after a prompt, and the picks the
    session entry point makes from them for every option set."""
    W = synth.make_weights(cfg, seed, std=0.08)
    gm = G.Model.from_tensors(cfg, W)
    gs = G.Session(gm, batch=batch)
    prompts = np.stack([synth.uniform_tokens(plen, cfg.vocab, seed + 1, stream=b) for b in range(batch)])
    prompts[:, -3] = prompts[:, -1]  # a repeated token inside the penalty window
    logits = gs.prefill(prompts)
    u = synth.uniforms(batch, seed + 2)
    want = [gs.pick(G.sampling(**o), uniforms=u).copy() for o in OPTIONS]
    # ... which are the CPU checker's own from the same logits, history and draws (text_gen.cpp:14-33,
    # :52-60, :135-209): the comparison below is with the reference's arithmetic, not only with the session's
    # (not the top-p walk over a whole vocabulary of 50 k nearly equal probabilities: there the rounding
    # of the running sum decides between neighbours, which the sampler's own tests hold to the checker
    # with their near-tie rule)
    for o, picks in zip(OPTIONS, want):
        if not o.get("greedy") and o.get("top_k", 0) == 0 and cfg.vocab > 10000:
            continue
        for b in range(batch):
            row = O.logits_with_penalty(logits[b], prompts[b], o.get("repetition_penalty", 1.0))
            ref = O.argmax_first(row) if o.get("greedy") else O.sample_from_logits(
                row, o.get("temperature", 1.0), o.get("top_k", 0), o.get("top_p", 1.0), float(u[b]))
            assert int(picks[b]) == int(ref), (o, b, int(picks[b]), int(ref))
    dev = dict(logits=torch.from_numpy(np.ascontiguousarray(logits)).cuda(),
               hist=torch.from_numpy(np.ascontiguousarray(prompts.astype(np.int32))).cuda(),
               u=torch.from_numpy(u.astype(np.float32)).cuda(),
               out=torch.full((len(OPTIONS), batch), -7, dtype=torch.int32, device="cuda"))
    return dev, want, batch, cfg.vocab, plen


def _run(torch, dev, batch, vocab, plen):
    for i, o in enumerate(OPTIONS):
        G.pick_noalloc(dev["logits"].data_ptr(), batch, vocab, dev["hist"].data_ptr(), plen, plen,
                       G.sampling(**o), dev["out"][i].data_ptr(), uniforms_ptr=dev["u"].data_ptr())
    torch.cuda.synchronize()
    return dev["out"].cpu().numpy()


def test_noalloc_pick_equals_session_pick_twice_in_a_row():
    torch = _torch_on_the_loaded_runtime()
    G.device_info()  # the documented set-up call: looks the scratch array up on this device
    big = _case(torch, synth.Config(synth.ARCH_MODERN, 50257, 128, 2, 2, 32), 900, 3, 12)
    small = _case(torch, synth.Config(synth.ARCH_GPT2, 777, 128, 2, 2, 32), 910, 1, 9)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]  # hipMemGetInfo: the device's own count, whoever allocates
    got_big = _run(torch, *[big[0]], *big[2:])
    got_small = _run(torch, *[small[0]], *small[2:])  # smaller rows over the first call's leftovers
    got_big2 = _run(torch, *[big[0]], *big[2:])
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    for i in range(len(OPTIONS)):
        assert np.array_equal(got_big[i], big[1][i]), (OPTIONS[i], got_big[i], big[1][i])
        assert np.array_equal(got_small[i], small[1][i]), (OPTIONS[i], got_small[i], small[1][i])
        assert np.array_equal(got_big2[i], big[1][i])


def test_noalloc_pick_under_stream_capture():
    """The callers the entry point is for: a stream under capture in global mode, where an
    allocation, a free or a wait inside a call ends the capture with an error.  The
    captured picks are replayed three times with eager work between the replays and must
    be the session's every time."""
    torch = _torch_on_the_loaded_runtime()
    G.device_info()
    dev, want, batch, vocab, plen = _case(torch, synth.Config(synth.ARCH_MODERN, 5000, 128, 2, 2, 32), 930, 2, 11)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        for i, o in enumerate(OPTIONS):
            G.pick_noalloc(dev["logits"].data_ptr(), batch, vocab, dev["hist"].data_ptr(), plen, plen,
                           G.sampling(**o), dev["out"][i].data_ptr(), uniforms_ptr=dev["u"].data_ptr(),
                           stream=side.cuda_stream)
    for _ in range(3):
        dev["out"].fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = dev["out"].cpu().numpy()
        for i in range(len(OPTIONS)):
            assert np.array_equal(got[i], want[i]), (OPTIONS[i], got[i], want[i])


def test_noalloc_pick_philox_draws_and_limits():
    torch = _torch_on_the_loaded_runtime()
    cfg = synth.Config(synth.ARCH_MODERN, 1000, 128, 2, 2, 32)
    W = synth.make_weights(cfg, 920, std=0.08)
    gs = G.Session(G.Model.from_tensors(cfg, W))
    prompt = synth.uniform_tokens(10, cfg.vocab, 921)
    logits = gs.prefill(prompt[None, :])
    opt = G.sampling(temperature=1.1, top_k=50, top_p=0.95, repetition_penalty=1.1)
    want = gs.pick(opt, seed=77)  # the session's first pick: draw index 0 of stream (77, sequence 0)
    lg = torch.from_numpy(np.ascontiguousarray(logits)).cuda()
    hist = torch.from_numpy(prompt.astype(np.int32)).cuda()
    out = torch.zeros(1, dtype=torch.int32, device="cuda")
    G.pick_noalloc(lg.data_ptr(), 1, cfg.vocab, hist.data_ptr(), 10, 10, opt, out.data_ptr(), seed=77, pick_index=0)
    torch.cuda.synchronize()
    assert int(out.cpu()[0]) == int(want[0])
    # beyond the array: refused with a clear message, nothing launched
    with pytest.raises(ValueError, match="exceed the 4 MiB scratch"):
        G.pick_noalloc(lg.data_ptr(), 64, 50257, hist.data_ptr(), 10, 10, opt, out.data_ptr())
    with pytest.raises(ValueError):
        G.pick_noalloc(lg.data_ptr(), 0, cfg.vocab, hist.data_ptr(), 10, 10, opt, out.data_ptr())
