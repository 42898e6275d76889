"""Decode throughput of the KV-cached token loop on one MI355X.

A step is one pass of the hot path over one batch: one new token for every
sequence (pick on the GPU, then the whole transformer step).  The default
workload is the 69M Llama block at batch 1 with the sampler the config names
(temperature 0.8, top-k 40, top-p 0.9, repetition penalty 1.1), timed over
--steps steps; the same workload as named (32 + 224), the two GPT-2 block
workloads, the 64-sequence batched decode and the 2048-context decode are reported
beside it, each with its fraction of the HBM roofline, and the CPU checker is timed
on every one of them.  Weights are seeded
N(0, 0.02), prompts seeded uniform ids; both live on the GPU before the clock
starts.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(ROOT, "grad.cpp_amd"), os.path.join(ROOT, "tests"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# HBM traffic of the batch-1 persistent kernel, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE of a 224-step launch at contexts 33..256 (the counters converted to bytes
# with the factors a 1 GiB copy kernel gives for them), as a ratio to the algorithmic
# bytes of the same launch.  The kernel reads every weight once per step whatever the
# number of steps, so the ratio carries over to other launch lengths; the summary named
# here holds the commands and the raw counts.
PMC_SOURCE = "profiles/persist_decode_kernel_c2_batch1.md"
PMC_FETCH_BYTES_PER_LAUNCH = 31_362_617 * 2048  # counter reads 1 per 2 KiB fetched
PMC_WRITE_BYTES_PER_LAUNCH = 556_358 * 1024     # counter reads 1 per KiB written
PMC_ALGORITHMIC_BYTES_PER_LAUNCH = 63_406_751_744  # step_bytes() summed over that launch


# Per-leg step times this tree is expected to reach on an MI355X (tracked next to the
# profiles they come from); the line reports measured / expected for every leg, and
# tests/test_gpu_regression.py fails beyond the file's tolerance.
EXPECTED_FILE = os.path.join(ROOT, "profiles", "expected_step_times.json")


def regression(line):
    """{leg: measured ms per step / expected} for the legs of a bench line."""
    try:
        expected = json.load(open(EXPECTED_FILE))["ms_per_step"]
    except (OSError, KeyError, ValueError):
        return None
    out = {}
    for leg, want in expected.items():
        got = line.get("ms_per_step") if leg == "c2" else (line.get(leg) or {}).get("ms_per_step")
        if got and want:
            out[leg] = round(got / want, 3)
    return out


def step_bytes(cfg, batch, ctx):
    """Algorithmic bytes of one decode step: every matrix once (regardless of
    batch), small vectors, the KV rows read at context `ctx` per sequence, the
    KV rows written, embedding rows and the logits written.  All fp32."""
    d, L, F, V = cfg.d_model, cfg.layers, cfg.d_ff, cfg.vocab
    mats = L * (4 * d * d + (3 if cfg.modern else 2) * d * F) + V * d
    vecs = L * (4 * d + 4 * d + (0 if cfg.modern else F + d)) + 2 * d
    kv_read = batch * L * 2 * ctx * d
    per_seq = L * 2 * d + d + (0 if cfg.modern else d) + V
    return 4 * (mats + vecs + kv_read + batch * per_seq)


def run_decode(G, synth, gm, cfg, batch, prompt_len, steps, warmup, opt, seed, engine, flags=0):
    """Times exactly `steps` decode steps (in rounds that fit the context) with
    the host clock around synchronised GPU work; returns totals."""
    gs = G.Session(gm, batch=batch, engine=engine, flags=flags)
    prompts = np.stack([synth.uniform_tokens(prompt_len, cfg.vocab, seed, stream=b) for b in range(batch)])
    room = cfg.max_len - prompt_len
    done = -warmup
    wall = gpu_ms = 0.0
    byte_sum = 0
    launches = []  # (steps, GPU ms, algorithmic bytes) of every timed decode round
    prefill_ms = 0.0
    prefill_tok = 0
    while done < steps:
        n = min(room, (steps - done) if done >= 0 else min(-done, room))
        gs.reset()
        t0 = time.perf_counter()
        gs.prefill(prompts)            # synchronous: returns the last logits
        t1 = time.perf_counter()
        picks = gs.decode(n, opt, seed=seed)  # synchronous
        t2 = time.perf_counter()
        tm = gs.last_timing()
        assert picks.shape == (batch, n)
        if done >= 0:
            wall += t2 - t1
            gpu_ms += tm["decode_ms"]
            round_bytes = sum(step_bytes(cfg, batch, prompt_len + i + 1) for i in range(n))
            byte_sum += round_bytes
            launches.append((n, tm["decode_ms"], round_bytes))
            prefill_ms += (t1 - t0) * 1e3
            prefill_tok += batch * prompt_len
        done += n
    return {"wall_s": wall, "gpu_ms": gpu_ms, "bytes": byte_sum, "steps": steps, "launches": launches,
            "launches_per_step": tm["launches_per_step"],
            "prefill_tok_s": prefill_tok / (prefill_ms / 1e3) if prefill_ms else None}


def _cpu_run(O, om, prompt, n_new, pick, thread_plan):
    """One sequence through the CPU checker, token by token like the reference's loop.
    thread_plan: [(first_step, threads)], applied when that step is reached.  Returns
    the seconds of every step() call."""
    sess = O.Session(om)
    plan = dict(thread_plan)
    secs = np.zeros(len(prompt) + n_new)
    toks = [int(t) for t in prompt]
    logits = None
    for i in range(len(prompt) + n_new):
        if i in plan:
            O.blas_set_threads(plan[i])
        t0 = time.perf_counter()
        if i >= len(prompt):
            toks.append(pick(logits, toks, i - len(prompt)))
        logits = sess.step(toks[i])
        secs[i] = time.perf_counter() - t0
    return secs


def cpu_baseline(synth, W2):
    """The CPU checker (a port of the reference's loop: one M=1 sgemm per projection,
    BLAS-backed like it) timed on this host at 1 BLAS thread and at all of them (16 at
    most), on every named workload.  The reference has no batch dimension, so c3 and c4
    are one sequence each and their rate is the rate of any number of sequences run one
    after another.  The pick is timed with the step it feeds."""
    import oracle_lib as O
    provider = O.blas_init()
    ncpu = len(os.sched_getaffinity(0))
    nt = min(ncpu, 16)
    opts = (0.8, 40, 0.9, 1.1)
    u = synth.uniforms(224, 3002)

    def greedy(penalty):
        return lambda lg, toks, i: int(O.argmax_first(O.logits_with_penalty(lg, np.asarray(toks, np.int32), penalty)
                                                      if penalty != 1.0 else lg))

    def sampled(lg, toks, i):
        adj = O.logits_with_penalty(lg, np.asarray(toks, np.int32), opts[3])
        return int(O.sample_from_logits(adj, opts[0], opts[1], opts[2], float(u[i])))

    out = {}
    # (name, weights preset, prompt, new tokens, pick, seed)
    plans = [("c0", "c0", 16, 80, greedy(1.2), 2000), ("c1", "c1", 32, 224, greedy(1.0), 2001),
             ("c2", "c2", 32, 224, sampled, 2002), ("c3", "c2", 128, 128, greedy(1.0), 2003)]
    for name, wname, n_prompt, n_new, pick, seed in plans:
        cfg = synth.PRESETS[wname]
        W = W2 if wname == "c2" else synth.make_weights(cfg, 1000 + int(wname[1]))
        om = O.Model.from_tensors(cfg, W)
        prompt = synth.uniform_tokens(n_prompt, cfg.vocab, seed)
        rates = {}
        for threads in (1, nt):
            secs = _cpu_run(O, om, prompt, n_new, pick, [(0, threads)])
            rates[threads] = {"prompt_tok_s": round(n_prompt / secs[:n_prompt].sum(), 2),
                              "decode_tok_s": round(n_new / secs[n_prompt:].sum(), 2)}
        out[name] = {"threads_1": rates[1], f"threads_{nt}": rates[nt],
                     "sample": f"one sequence in full: {n_prompt} prompt steps + {n_new} decode steps"
                               + ("; the reference runs the 64 sequences one after another at this rate"
                                  if name == "c3" else "")}
        del om
    # c4: one sequence of 1536 + 512 steps costs about a minute on one thread, so the
    # single-thread rate is taken on two windows of 32 steps (contexts 768.. and 2016..)
    # of a pass that otherwise runs on all threads.
    cfg4 = synth.PRESETS["c4"]
    om = O.Model.from_tensors(cfg4, W2)
    prompt = synth.uniform_tokens(1536, cfg4.vocab, 2004)
    secs = _cpu_run(O, om, prompt, 512, greedy(1.0), [(0, nt), (768, 1), (800, nt), (2016, 1)])
    many_prompt = np.r_[secs[:768], secs[800:1536]]
    out["c4"] = {"threads_1": {"prompt_tok_s": round(32 / secs[768:800].sum(), 2),
                               "decode_tok_s": round(32 / secs[2016:].sum(), 2)},
                 f"threads_{nt}": {"prompt_tok_s": round(len(many_prompt) / many_prompt.sum(), 2),
                                   "decode_tok_s": round(480 / secs[1536:2016].sum(), 2)},
                 "sample": "one sequence of 1536 prompt + 512 decode steps on all threads, except steps "
                           "768..799 (prompt) and 2016..2047 (decode), which run on one thread and give "
                           "the single-thread rates at those contexts; 16 sequences run one after another "
                           "at this rate"}
    del om
    O.blas_set_threads(nt)
    best = max((1, nt), key=lambda t: out["c2"][f"threads_{t}"]["decode_tok_s"])
    return {"value": out["c2"][f"threads_{best}"]["decode_tok_s"], "unit": "tok/s", "cores": best, "kind": "port",
            "sample": "decode steps of the headline workload (c2: 32 prompt steps, then 224 sampled decode "
                      f"steps), one pass per thread setting; BLAS: {provider.split(' [')[0].split('/')[-1]}",
            "single_thread": out["c2"]["threads_1"]["decode_tok_s"], "host_cpus": ncpu, "configs": out}


def phase_stamps(xcd=False, greedy=False, row_picks=False):
    """Mean phase durations of one token of c2 on a persistent kernel, from the stamps
    workgroup 0 leaves (GRADHIP_PROF_DUMP).  The all-to-all kernel: per step one stamp
    after the pick, five per layer, one when the logits rows have arrived, one at the
    end.  The XCD-sharded kernel: one after the pick, eight per layer (a phase's
    arithmetic, then the wait for the next phase's operands), one at the end."""
    import tempfile
    dump = os.path.join(tempfile.mkdtemp(), "stamps.txt")
    os.environ["GRADHIP_PROF_DUMP"] = dump
    import gradhip as G
    from gradhip import synth
    cfg = synth.PRESETS["c2"]
    gm = G.Model.from_tensors(cfg, synth.make_weights(cfg, 1002))
    gs = G.Session(gm, engine=G.ENGINE_PERSISTENT,
                   flags=(G.FLAG_XCD_PERSISTENT if xcd else G.FLAG_CLASSIC_PERSISTENT)
                   | (G.FLAG_ROW_PICKS if row_picks else 0))
    gs.prefill(synth.uniform_tokens(32, cfg.vocab, 2002)[None, :])
    gs.decode(224, G.sampling(greedy=True, repetition_penalty=1.0) if greedy else G.sampling(0.8, 40, 0.9, 1.1),
              seed=2002)
    gpu_us = gs.last_timing()["decode_ms"] * 1e3 / 224
    gs.close()  # writes the dump: stamps, "0", three clock readings per pick, "0", counters
    words = open(dump).read().split()
    z = words.index("0")
    z2 = words.index("0", z + 1)
    st = np.array([int(x) for x in words[:z]], dtype=np.float64) / 100.0  # 100 MHz clock -> us
    L = cfg.layers
    per_layer = 8 if xcd else 5
    period = per_layer * L + (2 if xcd else 3)
    d = np.diff(st)
    k = len(d) // period - 3
    m = d[2 * period: (2 + k) * period].reshape(k, period).mean(axis=0)
    lay = m[1:1 + per_layer * L].reshape(L, per_layer).mean(axis=0)
    pk = np.array([int(x) for x in words[z + 1:z2]], dtype=np.float64) / 100.0
    pk = pk[: len(pk) // 3 * 3].reshape(-1, 3)[3:]
    out = {
        "workload": "c2%s, one launch of 224 pick + step rounds, contexts 33..256" % (" with greedy picks" if greedy else ""),
        "steps_averaged": int(k),
        "kernel": "xcd_decode_kernel" if xcd else "persist_decode_kernel",
        "us_per_token_events": round(gpu_us, 2), "us_per_token_stamps": round(float(m.sum()), 2),
        "pick_until_token_seen": round(float(m[0]), 2),
        "pick_inside": {"wait_for_logits": round(float((pk[:, 1] - pk[:, 0]).mean()), 2),
                        "penalty_sampler_token_out": round(float((pk[:, 2] - pk[:, 1]).mean()), 2)}}
    if xcd:
        names = ["norm1+qkv_rows", "wait_attention_partials", "merge+w_o_partials", "wait_x_after_attention",
                 "norm2+gate_up_rows", "wait_hidden", "w_down_partials", "wait_x_of_next_layer"]
        out["layer_mean"] = {n: round(float(v), 2) for n, v in zip(names, lay)}
        out["layer_mean"]["sum"] = round(float(lay.sum()), 2)
        out["layers_total"] = round(float(lay.sum() * L), 2)
        out["logits_rows_from_the_ring"] = round(float(m[-1]), 2)
        tail = [int(x) for x in words[z2 + 1:]]
        # polls that found the ring not yet filled, per token (stored + 1): P1, P3, P5, P6, logits
        out["ring_stall_polls_per_token"] = [round((v - 1) / 224.0, 2) for v in tail[96:101] if v > 0]
    else:
        out["layer_mean"] = {"embed_or_x_exchange+norm1+qkv": round(float(lay[0]), 2),
                             "qkv_exchange+attention": round(float(lay[1]), 2),
                             "attn_exchange+w_o": round(float(lay[2]), 2),
                             "x_exchange+norm2+ffn1": round(float(lay[3]), 2),
                             "hidden_exchange+ffn2": round(float(lay[4]), 2), "sum": round(float(lay.sum()), 2)}
        out["layers_total"] = round(float(lay.sum() * L), 2)
        out["x_exchange+logits_rows_arrive"] = round(float(m[-2]), 2)
        out["logits_dots_stores_arrival_count"] = round(float(m[-1]), 2)
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=448)
    ap.add_argument("--warmup", type=int, default=224)
    ap.add_argument("--engine", default="auto", choices=["auto", "graph", "eager", "persistent"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-batch64", action="store_true", help="skip the batch-64 leg")
    ap.add_argument("--no-small", action="store_true", help="skip the c0, c1 and c2-as-named legs")
    ap.add_argument("--only-batch64", action="store_true",
                    help="run only the batch-64 leg and print its object (for profiling that leg alone)")
    ap.add_argument("--no-long", action="store_true", help="skip the 2048-context leg")
    ap.add_argument("--only-long", action="store_true",
                    help="run only the 2048-context leg and print its object (for profiling that leg alone)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run a 1 GiB device-to-device copy three times (calibrates rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters against a kernel of known traffic) and exit")
    ap.add_argument("--stream-probe", action="store_true",
                    help="only time a plain read of 2 GiB (what a streaming kernel can reach of the "
                         "published HBM peak on this device) and exit")
    ap.add_argument("--cache-probe", action="store_true",
                    help="only time back-to-back re-reads of buffers from 32 MiB to 2 GiB (shows up to which "
                         "size the memory-side cache serves a re-read) and exit")
    ap.add_argument("--phase-stamps", action="store_true",
                    help="only run one 224-step launch of the batch-1 workload with the persistent kernel's "
                         "in-kernel phase stamps on (workgroup 0's clock at the end of every phase) and "
                         "print the mean duration of every phase of a token")
    ap.add_argument("--row-picks", action="store_true",
                    help="batch-1 legs and --phase-stamps: every pick by one workgroup from the whole row of "
                         "logits (GH_FLAG_ROW_PICKS) instead of by every workgroup from candidates")
    ap.add_argument("--greedy-picks", action="store_true",
                    help="with --phase-stamps: greedy picks without a penalty instead of the workload's sampler")
    ap.add_argument("--kernel", default="auto", choices=["auto", "classic", "xcd"],
                    help="pin the batch-1 legs to one of the persistent engine's two kernels (the all-to-all "
                         "kernel or the XCD-sharded one); auto: by position, as sessions do by default")
    ap.add_argument("--step-loop", action="store_true",
                    help="only time the literal drop-in loop on the batch-1 workload: one InferenceSession::step "
                         "call per token (one launch and one copy of the logits to the host each) with the "
                         "arg-max on the host, as text_gen.cpp:44-64 does, and exit")
    ap.add_argument("--handoff-probe", action="store_true",
                    help="only time a two-workgroup ping-pong (same XCD / two XCDs, ordinary or device-scope "
                         "stores, non-temporal or device-scope loads, idle or beside 240 streaming workgroups) "
                         "and exit")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="only time fp32 matrix products and ordinary multiply-adds on the same SIMDs, apart and "
                         "together (does anything issue beside a running product?), and exit")
    ap.add_argument("--phase-stamps-xcd", action="store_true",
                    help="the same for the XCD-sharded persistent kernel (eight stamps per layer)")
    a = ap.parse_args()
    if a.phase_stamps or a.phase_stamps_xcd:
        phase_stamps(xcd=a.phase_stamps_xcd, greedy=a.greedy_picks, row_picks=a.row_picks)
        return
    if a.handoff_probe:
        import gradhip as G
        rows = []
        for busy in (False, True):
            for peer in (8, 1):
                for store_dev, load, name in ((True, 2, "device-scope store, device-scope load"),
                                              (True, 1, "device-scope store, non-temporal load"),
                                              (False, 1, "ordinary store, non-temporal load"),
                                              (False, 2, "ordinary store, device-scope load")):
                    us, xa, xb = G.handoff_latency(load, store_dev, peer, busy)
                    rows.append({"busy": busy, "xcds": [xa, xb], "policy": name, "us_per_round_trip": round(us, 3)})
        print(json.dumps({"handoff": rows}))
        return
    if a.mfma_probe:
        import gradhip as G
        rows = []
        for per in (8, 16, 24):
            for mode, name in ((1, "products alone (wavefronts 0-3)"), (2, "multiply-adds alone (wavefronts 4-7)"),
                               (3, "both, on the same SIMDs"), (4, "one wavefront per SIMD doing both in turn")):
                if mode == 1 and per != 8:
                    continue
                prod, slot, mhz = G.mfma_issue(mode, per)
                rows.append({"multiply_adds_per_slot": per, "what": name, "clk_per_product": round(prod, 1),
                             "clk_per_slot": round(slot, 1), "shader_mhz": round(mhz)})
        print(json.dumps({"mfma_issue": rows}))
        return
    if a.cache_probe:
        import gradhip as G
        rows = []
        for mib in (1, 8, 32, 64, 96, 128, 160, 192, 224, 256, 288, 320, 384, 512, 768, 1024, 2048):
            passes = max(8, min(200, (16 << 10) // mib))
            rate = G.reread_bandwidth(mib << 20, passes)
            rows.append({"MiB": mib, "passes": passes, "GBps": round(rate, 1),
                         "us_per_pass": round((mib << 20) / rate / 1e3, 2)})
        print(json.dumps({"reread": rows}))
        return
    if a.stream_probe:
        import gradhip as G
        best = G.read_bandwidth(2 << 30, 5)
        print(json.dumps({"stream_read_GBps": round(best, 1), "peak_GBps": HBM_PEAK_GBS,
                          "frac": round(best / HBM_PEAK_GBS, 3)}))
        return
    if a.copy_probe:
        import torch
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_bytes_read": 1 << 30, "copy_probe_bytes_written": 1 << 30}))
        return
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (more GPUs would each take a share of the "
                 "sequences, with the weights replicated and nothing exchanged); run with --gpus 1")

    import gradhip as G
    from gradhip import synth
    info = G.device_info()
    engine = {"auto": G.ENGINE_AUTO, "graph": G.ENGINE_GRAPH, "eager": G.ENGINE_EAGER,
              "persistent": G.ENGINE_PERSISTENT}[a.engine]

    cfg = synth.PRESETS["c2"]
    W = synth.make_weights(cfg, 1002)
    gm = G.Model.from_tensors(cfg, W)
    opts = (0.8, 40, 0.9, 1.1)
    sample = G.sampling(*opts)

    b1_flags = {"auto": 0, "classic": G.FLAG_CLASSIC_PERSISTENT, "xcd": G.FLAG_XCD_PERSISTENT}[a.kernel]
    if a.row_picks:
        b1_flags |= G.FLAG_ROW_PICKS
    if a.step_loop:
        gs = G.Session(gm, engine=engine, flags=b1_flags)
        prompt = synth.uniform_tokens(32, cfg.vocab, 2002)
        best = None
        for rep in range(3):
            gs.reset()
            logits = gs.prefill(prompt[None, :])[0]
            t0 = time.perf_counter()
            for _ in range(224):
                logits = gs.step([int(np.argmax(logits))])[0]
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        print(json.dumps({"workload": "c2, 32-token prompt, 224 x (host arg-max + step() with the logits copied "
                                      "to the host)", "value": round(224 / best, 1), "unit": "tok/s",
                          "us_per_token": round(best * 1e6 / 224, 2), "kernel": a.kernel,
                          "launches_per_step": gs.last_timing()["launches_per_step"]}), flush=True)
        return
    if a.only_batch64:
        greedy = G.sampling(greedy=True, repetition_penalty=1.0)
        r64 = run_decode(G, synth, gm, cfg, 64, 128, 128, 16, greedy, 2003, engine)
        print(json.dumps({"workload": "c3", "value": round(64 * r64["steps"] / r64["wall_s"], 1), "unit": "tok/s",
                          "us_per_step_gpu": round(r64["gpu_ms"] * 1e3 / r64["steps"], 2)}), flush=True)
        return
    if a.only_long:
        cfg4 = synth.PRESETS["c4"]
        gm4 = G.Model.from_tensors(cfg4, W)
        greedy = G.sampling(greedy=True, repetition_penalty=1.0)
        r4 = run_decode(G, synth, gm4, cfg4, 16, 1536, 512, 16, greedy, 2004, engine)
        print(json.dumps({"workload": "c4", "value": round(16 * r4["steps"] / r4["wall_s"], 1), "unit": "tok/s",
                          "us_per_step_gpu": round(r4["gpu_ms"] * 1e3 / r4["steps"], 2),
                          "prefill_tok_s": round(r4["prefill_tok_s"], 1)}), flush=True)
        return
    def roofline(r):
        ach = r["bytes"] / (r["gpu_ms"] / 1e3) / 1e9
        return {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(ach / HBM_PEAK_GBS, 4)}

    def leg(workload, r, batch):
        return {"workload": workload, "value": round(batch * r["steps"] / r["wall_s"], 1), "unit": "tok/s",
                "ms_per_step": round(r["wall_s"] * 1e3 / r["steps"], 5),
                "prefill_tok_s": round(r["prefill_tok_s"], 1), "roofline": roofline(r)}

    r1 = run_decode(G, synth, gm, cfg, 1, 32, a.steps, a.warmup, sample, 2002, engine, b1_flags)
    tok_s = r1["steps"] / r1["wall_s"]
    persistent = r1["launches_per_step"] == 1
    n_l = len(r1["launches"])
    us_per_launch = sum(ms for _, ms, _ in r1["launches"]) * 1e3 / n_l
    bytes_per_launch = sum(nb for _, _, nb in r1["launches"]) / n_l
    steps_per_launch = sum(n for n, _, _ in r1["launches"]) / n_l
    achieved = bytes_per_launch / (us_per_launch * 1e-6) / 1e9
    if persistent:
        # template arguments: d_model / 256, FFN width / 256, Llama block, sampler row in LDS (vocabularies
        # up to ~38 k), not the streaming variant
        kernel = (f"gh::persist_decode_kernel<{cfg.d_model // 256}, {cfg.d_ff // 256}, "
                  f"{'true' if cfg.modern else 'false'}, {'true' if cfg.vocab <= 38000 else 'false'}, false>: "
                  "one launch = one pick + step round per token for a whole run of steps")
        if a.kernel == "xcd":
            kernel = ("gh::xcd_decode_kernel<3, true, false>: the XCD-sharded persistent kernel, one launch = one "
                      "pick + step round per token for a whole run of steps")
        # measured HBM bytes per algorithmic byte of this kernel, times this launch's algorithmic bytes
        traffic = int(bytes_per_launch * (PMC_FETCH_BYTES_PER_LAUNCH + PMC_WRITE_BYTES_PER_LAUNCH)
                      / PMC_ALGORITHMIC_BYTES_PER_LAUNCH)
        traffic_source = (f"{PMC_SOURCE}: FETCH_SIZE + WRITE_SIZE of a 224-step launch of this kernel are "
                          f"{(PMC_FETCH_BYTES_PER_LAUNCH + PMC_WRITE_BYTES_PER_LAUNCH) / PMC_ALGORITHMIC_BYTES_PER_LAUNCH:.4f}"
                          " of its algorithmic bytes; scaled to this launch's algorithmic bytes")
    else:
        kernel = "every kernel of the decode round (one launch per fused op), timed as one span"
        traffic = None
        traffic_source = "no counter run covers this engine"

    line = {
        "metric": "decode tok/s, 69M Llama block, batch 1",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(r1["wall_s"] * 1e3 / r1["steps"], 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c2: Llama block 69M (d768 L8 H12 F2048 V16000 C256), batch 1, "
                               "32-token prompt, sampled decode T0.8 top-k40 top-p0.9 penalty1.1",
                   "batch": 1, "engine": a.engine, "launches_per_step": r1["launches_per_step"]},
        "device": info["name"],
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": traffic_source,
                     "traffic_is": "this launch's algorithmic bytes times the HBM-to-algorithmic ratio that "
                                   "rocprofv3 --pmc measured on a 224-step launch of the same kernel; not "
                                   "re-measured in this run" if traffic is not None else None,
                     "kernel": kernel, "launches": n_l, "steps_per_launch": steps_per_launch,
                     "us_per_launch": round(us_per_launch, 1),
                     "bytes_per_launch": int(bytes_per_launch)},
        "prefill_tok_s": round(r1["prefill_tok_s"], 1),
    }
    # what a plain streaming-read kernel reaches on this device, measured now: the
    # practical ceiling the published peak has to be read against
    stream = G.read_bandwidth(2 << 30, 5)
    line["roofline"]["stream_read"] = round(stream, 1)
    line["roofline"]["frac_of_stream_read"] = round(achieved / stream, 4)

    greedy = G.sampling(greedy=True, repetition_penalty=1.0)
    if not a.no_small:
        # the workload exactly as named, whatever --steps says: 32 prompt tokens, 224 sampled steps
        rf = run_decode(G, synth, gm, cfg, 1, 32, 224, 224, sample, 2002, engine, b1_flags)
        line["c2_full"] = leg("c2 as named: 32-token prompt, then 224 sampled decode steps (one launch)", rf, 1)
        # c0 (the shape of the reference's own published figure) and c1
        cfg0 = synth.PRESETS["c0"]
        gm0 = G.Model.from_tensors(cfg0, synth.make_weights(cfg0, 1000))
        r0 = run_decode(G, synth, gm0, cfg0, 1, 16, 80, 80, G.sampling(greedy=True, repetition_penalty=1.2),
                        2000, engine, b1_flags & G.FLAG_ROW_PICKS)
        line["c0"] = leg("c0: GPT-2 block 'small' (d512 L6 H8 F2048 V5000 C96), batch 1, 16-token prompt, "
                         "80 greedy steps, repetition penalty 1.2 (the reference's default)", r0, 1)
        del gm0
        cfg1 = synth.PRESETS["c1"]
        gm1 = G.Model.from_tensors(cfg1, synth.make_weights(cfg1, 1001))
        r1m = run_decode(G, synth, gm1, cfg1, 1, 32, 224, 224, greedy, 2001, engine, b1_flags & G.FLAG_ROW_PICKS)
        line["c1"] = leg("c1: GPT-2 block 'medium' (d768 L8 H12 F3072 V16000 C256), batch 1, 32-token prompt, "
                         "224 greedy steps", r1m, 1)
        del gm1

    if not a.no_small:
        # The reference's own published protocol for this path (src/cli/bench.cpp:269-286):
        # five timed calls of generate_sample(prompt, temperature 0.8, 64 tokens) with
        # TextGen's defaults (penalty 1.2, no top-k / top-p) on the 'small' GPT-2 shape with
        # the presets' context of 1024, a fresh session per call, host wall time including
        # the session's construction and the prompt steps; median of 64 / seconds.  Its
        # published figures: 385.1 tok/s (M2 Pro), 843.5 / 854.5 (M3 Pro).
        cfgb = synth.Config(synth.ARCH_GPT2, 5000, 512, 6, 8, 1024)
        gmb = G.Model.from_tensors(cfgb, synth.make_weights(cfgb, 1000))
        prompt_b = np.frombuffer(b"ROMEO:\n", dtype=np.uint8).astype(np.int32)[None, :]
        rates = []
        for trial in range(6):
            t0 = time.perf_counter()
            sb = G.Session(gmb)
            toks = sb.generate(prompt_b, 64, G.sampling(0.8, 0, 1.0, 1.2), seed=trial)
            sb.close()
            dt = time.perf_counter() - t0
            assert toks.shape[1] == prompt_b.shape[1] + 64
            if trial:  # the first call also loads the kernels' code: a warm-up, like a first run of the binary
                rates.append(64.0 / dt)
        line["grad_bench_protocol"] = {
            "workload": "grad bench's generation figure: GPT-2 'small' (d512 L6 H8 V5000 C1024), 7-token prompt, "
                        "generate_sample(T 0.8, 64 tokens, penalty 1.2), fresh session per call, wall time "
                        "including session construction; median of 5 calls after one warm-up call",
            "value": round(float(np.median(rates)), 1), "unit": "tok/s", "trials": [round(r, 1) for r in rates],
            "reference_published": {"M2 Pro": 385.1, "M3 Pro": [843.5, 854.5]}}
        del gmb
        # Batch 1 at the context every preset of the reference ships (max_len 1024): the c2
        # weights, a 256-token prompt, greedy to the end of the context.
        cfgl = synth.Config(cfg.arch, cfg.vocab, cfg.d_model, cfg.layers, cfg.heads, 1024)
        gml = G.Model.from_tensors(cfgl, W)
        rl = run_decode(G, synth, gml, cfgl, 1, 256, 768, 768, greedy, 2002, engine, b1_flags)
        line["c2_ctx1024"] = leg("c2 weights with max_len 1024 (the reference presets' context), batch 1, "
                                 "256-token prompt, 768 greedy steps to the end of the context", rl, 1)
        del gml

    if not a.no_batch64:
        r64 = run_decode(G, synth, gm, cfg, 64, 128, 128, 16, greedy, 2003, engine)
        line["batch64"] = leg("c3: same model, 64 sequences, 128-token prompts, 128 greedy steps", r64, 64)

    if not a.no_long:
        # c4: same tensors, context 2048 (RoPE needs no table), 16 sequences with
        # 1536-token prompts in one pass, then greedy decode steps
        cfg4 = synth.PRESETS["c4"]
        gm4 = G.Model.from_tensors(cfg4, W)
        r4 = run_decode(G, synth, gm4, cfg4, 16, 1536, 512, 16, greedy, 2004, engine)
        line["context2048"] = leg("c4: same weights, context 2048, 16 sequences, 1536-token prompts "
                                  "in one pass, 512 greedy steps", r4, 16)
        del gm4

    line["regression"] = regression(line)
    line["cpu_baseline"] = None if a.no_cpu else cpu_baseline(synth, W)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
