"""The header-only C++ adapter (include/gradhip.hpp): a C++ caller written like
grad.cpp's generate/chat commands, compiled with g++ against the C ABI, must see
the same dims, logits, token streams, loop counts and exception types/messages."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as O
from gradhip import LIB_PATH, synth
from helpers import lively_std

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _build(tmp_path):
    exe = str(tmp_path / "adapter_test")
    lib_dir = os.path.dirname(LIB_PATH)
    subprocess.check_call(["g++", "-std=c++20", "-O1", "-Wall", "-Wextra", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "cpp", "adapter_test.cpp"), "-o", exe,
                           "-L", lib_dir, "-lgradhip", f"-Wl,-rpath,{lib_dir}"])
    return exe


@pytest.mark.parametrize("arch", [synth.ARCH_GPT2, synth.ARCH_MODERN])
def test_cpp_caller_matches_the_oracle(tmp_path, arch):
    cfg = synth.Config(arch, 301, 128, 2, 2, 40)
    W = synth.make_weights(cfg, 11, std=lively_std(cfg), norm_noise=0.1)
    path = str(tmp_path / "m.bin")
    synth.write_checkpoint(path, cfg, W, fingerprint=(2, 0xABCDEF))
    prompt = [int(t) for t in synth.uniform_tokens(6, cfg.vocab, 3)]
    exe = _build(tmp_path)
    out = subprocess.run([exe, path] + [str(t) for t in prompt], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    lines = {l.split(" ", 1)[0]: l.split(" ", 1)[1] if " " in l else "" for l in out.stdout.strip().split("\n")}
    assert "FATAL" not in lines, out.stdout
    assert lines["dims"].split() == [str(x) for x in (301, 128, 2, 2, 40, arch)]

    om = O.Model.from_tensors(cfg, W)
    s = O.Session(om)
    for t in prompt:
        ref = s.step(t)
    f = lines["step"].split()
    assert f[:3] == ["6", "40", "301"]
    got = np.array([float(x) for x in f[3:]])
    assert np.abs(got - ref[:8]).max() <= 1e-4 * np.abs(ref).max()
    assert out.stdout.count("out_of_range InferenceSession: token id out of vocab range") == 1
    assert out.stdout.count("runtime_error InferenceSession: context exceeds max_len") == 1

    greedy = O.generate_greedy(om, prompt, 12, 1.2)
    assert [int(x) for x in lines["greedy"].split()] == greedy.tolist()
    # sampled with the on-device Philox stream of seed 77: the same draws through the oracle
    u = synth.uniforms(12, 77)
    sampled = O.generate_sample(om, prompt, u, 0.8, 12, 1.1, 5, 0.9)
    assert [int(x) for x in lines["sample"].split()] == sampled.tolist()
    st = lines["stream"].split()
    assert int(st[0]) == 12 and [int(x) for x in st[1:]] == sampled.tolist()[len(prompt):]
    assert lines["callback_error"] == "third token"
    tail = sampled.tolist()[len(prompt):]
    cut = tail[:tail.index(tail[4]) + 1]  # ends after the first pick of the stop token
    sp = lines["stopped"].split()
    assert int(sp[0]) == len(cut) and [int(x) for x in sp[1:]] == cut
    assert lines["empty"] == "[]"
    over = O.generate_greedy(om, prompt, cfg.max_len + 10, 1.0)
    assert len(over) == cfg.max_len + 1  # the pick after the last step is pushed, then the loop stops
    assert [int(x) for x in lines["overflow"].split()] == over.tolist()
    assert lines["bytes"] == str(len(prompt) + 4)
    assert lines["load_error"] == "Could not open checkpoint for reading: /nonexistent/model.bin"
