"""Decode throughput of the KV-cached token loop on one MI355X.

A step is one pass of the hot path over one batch: one new token for every
sequence (pick on the GPU, then the whole transformer step).  The default
workload is the 69M Llama block at batch 1 with the sampler the config names
(temperature 0.8, top-k 40, top-p 0.9, repetition penalty 1.1); the 64-sequence
batched decode of the same model is reported beside it.  Weights are seeded
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

# rocprofv3 counters for one 224-step launch of the batch-1 persistent kernel
# (32-token prompt already cached): FETCH_SIZE and WRITE_SIZE, converted to bytes
# with the factors a 1 GiB copy kernel gives for the same counters.
PMC_STEPS_PER_LAUNCH = 224
PMC_FETCH_BYTES_PER_LAUNCH = 31_344_830 * 2048  # counter reads 1 per 2 KiB fetched
PMC_WRITE_BYTES_PER_LAUNCH = 541_326 * 1024     # counter reads 1 per KiB written


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


def run_decode(G, synth, gm, cfg, batch, prompt_len, steps, warmup, opt, seed, engine):
    """Times exactly `steps` decode steps (in rounds that fit the context) with
    the host clock around synchronised GPU work; returns totals."""
    gs = G.Session(gm, batch=batch, engine=engine)
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


def cpu_baseline(synth, cfg, W, prompt, uniforms, opts):
    """The CPU checker (a port of the reference's loop, BLAS-backed like it) timed
    on this host: the full batch-1 workload once per thread setting."""
    import oracle_lib as O
    provider = O.blas_init()
    om = O.Model.from_tensors(cfg, W)
    T, k, p, pen = opts
    out = {}
    ncpu = len(os.sched_getaffinity(0))
    for threads in (1, min(ncpu, 16)):
        O.blas_set_threads(threads)
        t0 = time.perf_counter()
        toks = O.generate_sample(om, prompt, uniforms, T, len(uniforms), pen, k, p)
        dt = time.perf_counter() - t0
        out[threads] = (len(toks)) / dt  # every step() call, prompt and decode alike
    best = max(out, key=out.get)
    return {"value": round(out[best], 2), "unit": "tok/s", "cores": best, "kind": "port",
            "sample": f"32 prompt + {len(uniforms)} sampled decode steps of the batch-1 workload, "
                      f"single pass per thread setting; BLAS: {provider.split(' [')[0].split('/')[-1]}",
            "single_thread": round(out[1], 2), "host_cpus": ncpu}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=448)
    ap.add_argument("--warmup", type=int, default=224)
    ap.add_argument("--engine", default="auto", choices=["auto", "graph", "eager", "persistent"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-batch64", action="store_true", help="skip the batch-64 leg")
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
    a = ap.parse_args()
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
    r1 = run_decode(G, synth, gm, cfg, 1, 32, a.steps, a.warmup, sample, 2002, engine)
    tok_s = r1["steps"] / r1["wall_s"]
    persistent = r1["launches_per_step"] == 1
    n_l = len(r1["launches"])
    us_per_launch = sum(ms for _, ms, _ in r1["launches"]) * 1e3 / n_l
    bytes_per_launch = sum(nb for _, _, nb in r1["launches"]) / n_l
    steps_per_launch = sum(n for n, _, _ in r1["launches"]) / n_l
    achieved = bytes_per_launch / (us_per_launch * 1e-6) / 1e9
    if persistent:
        kernel = ("gh::persist_decode_kernel<3, 8, true, true, false>: one launch = one pick + step round per token "
                  "for a whole run of steps")
    else:
        kernel = "every kernel of the decode round (one launch per fused op), timed as one span"
    # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (see the
    # summary under profiles/ for the command and the copy-kernel calibration);
    # only valid for the launch shape it was measured on.
    traffic = None
    if persistent and steps_per_launch == PMC_STEPS_PER_LAUNCH:
        traffic = PMC_FETCH_BYTES_PER_LAUNCH + PMC_WRITE_BYTES_PER_LAUNCH

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

    if not a.no_batch64:
        greedy = G.sampling(greedy=True, repetition_penalty=1.0)
        r64 = run_decode(G, synth, gm, cfg, 64, 128, 128, 16, greedy, 2003, engine)
        ach64 = r64["bytes"] / (r64["gpu_ms"] / 1e3) / 1e9
        line["batch64"] = {"workload": "c3: same model, 64 sequences, 128-token prompts, 128 greedy steps",
                           "value": round(64 * r64["steps"] / r64["wall_s"], 1), "unit": "tok/s",
                           "ms_per_step": round(r64["wall_s"] * 1e3 / r64["steps"], 4),
                           "prefill_tok_s": round(r64["prefill_tok_s"], 1),
                           "roofline": {"bound": "hbm", "achieved": round(ach64, 1), "peak": HBM_PEAK_GBS,
                                        "unit": "GB/s", "frac": round(ach64 / HBM_PEAK_GBS, 4)}}

    if not a.no_long:
        # c4: same tensors, context 2048 (RoPE needs no table), 16 sequences with
        # 1536-token prompts in one pass, then greedy decode steps
        cfg4 = synth.PRESETS["c4"]
        gm4 = G.Model.from_tensors(cfg4, W)
        greedy = G.sampling(greedy=True, repetition_penalty=1.0)
        r4 = run_decode(G, synth, gm4, cfg4, 16, 1536, 512, 16, greedy, 2004, engine)
        ach4 = r4["bytes"] / (r4["gpu_ms"] / 1e3) / 1e9
        line["context2048"] = {"workload": "c4: same weights, context 2048, 16 sequences, 1536-token prompts "
                                           "in one pass, 512 greedy steps",
                               "value": round(16 * r4["steps"] / r4["wall_s"], 1), "unit": "tok/s",
                               "ms_per_step": round(r4["wall_s"] * 1e3 / r4["steps"], 4),
                               "prefill_tok_s": round(r4["prefill_tok_s"], 1),
                               "roofline": {"bound": "hbm", "achieved": round(ach4, 1), "peak": HBM_PEAK_GBS,
                                            "unit": "GB/s", "frac": round(ach4 / HBM_PEAK_GBS, 4)}}
        del gm4

    if not a.no_cpu:
        prompt = synth.uniform_tokens(32, cfg.vocab, 2002)
        line["cpu_baseline"] = cpu_baseline(synth, cfg, W, prompt, synth.uniforms(224, 3002), opts)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
