"""Text in, text out: gradhip-generate (the `grad generate`-shaped caller, grad.cpp
src/cli/generate.cpp:61-107) encodes a prompt with a GTOK file, runs both loops on the
GPU and prints decoded text.  Checked against the CPU restatements of the tokenizer and
of the token loop; the tokenizer fingerprint guard against src/cli/common.cpp:254-268."""
import os
import subprocess
import sys

import pytest

import oracle_lib as O
from gradhip import synth
from helpers import lively_std

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import tokenizer_ref as R  # noqa: E402

CLI = os.path.join(ROOT, "grad.cpp_amd", "bin", "gradhip-generate")
TEXT = "Once upon a time, the little cat said: don't go!\nThe end. "


@pytest.fixture(scope="module")
def setup(tmp_path_factory):
    d = tmp_path_factory.mktemp("cli")
    tok = R.train((TEXT * 3 + "the cat sat on the mat and the cat ran to the hat\n" * 5).encode(), 330)
    (d / "t.tok").write_bytes(tok.file_image())
    cfg = synth.Config(synth.ARCH_MODERN, tok.vocab_size, 128, 2, 2, 64)
    W = synth.make_weights(cfg, 31, std=lively_std(cfg), norm_noise=0.1)
    synth.write_checkpoint(str(d / "m.bin"), cfg, W, fingerprint=(2, tok.fingerprint()))
    synth.write_checkpoint(str(d / "other.bin"), cfg, W, fingerprint=(2, tok.fingerprint() ^ 1))
    synth.write_checkpoint(str(d / "plain.bin"), cfg, W)
    return d, tok, cfg, O.Model.from_tensors(cfg, W)


def run(*args):
    assert os.path.exists(CLI), "gradhip-generate is not built; run __graft_entry__.build()"
    return subprocess.run([CLI, *[str(a) for a in args]], capture_output=True, timeout=120)


def test_generate_prints_the_oracles_text(setup):
    d, tok, cfg, om = setup
    prompt = "the little cat"
    out = run(d / "m.bin", d / "t.tok", prompt, "--max-tokens", 12, "--temperature", 0.8, "--top-k", 5, "--top-p",
              0.9, "--repetition-penalty", 1.1, "--seed", 77)
    assert out.returncode == 0, out.stdout + out.stderr
    ids = tok.encode(prompt.encode())
    greedy = O.generate_greedy(om, ids, 12, 1.1)
    sampled = O.generate_sample(om, ids, synth.uniforms(12, 77), 0.8, 12, 1.1, 5, 0.9)
    want = (b"\ngradhip Generation\n\n"
            + f"Tokenizer: {d / 't.tok'} (v2, vocab {tok.vocab_size})\n".encode()
            + b"\n--- Greedy Decoding ---\n\n" + f'Prompt: "{prompt}"\n'.encode() + tok.decode(greedy) + b"\n"
            + b"\n--- Sampling (temp=0.8, top-k=5, top-p=0.9) ---\n\n" + f'Prompt: "{prompt}"\n'.encode()
            + tok.decode(sampled) + b"\n")
    assert out.stdout == want
    only = run(d / "m.bin", d / "t.tok", prompt, "--max-tokens", 12, "--repetition-penalty", 1.1, "--greedy")
    assert only.returncode == 0 and b"Sampling" not in only.stdout and tok.decode(greedy) in only.stdout


def test_fingerprint_guard_and_exit_codes(setup):
    d, tok, cfg, om = setup
    out = run(d / "other.bin", d / "t.tok", "the cat")
    assert out.returncode == 1
    fp = tok.fingerprint()
    assert (f"Error: tokenizer v2:{fp:016x} is not the one {d / 'other.bin'} was trained with "
            f"(v2:{fp ^ 1:016x}); its token ids would mean different text").encode() in out.stderr
    out = run(d / "plain.bin", d / "t.tok", "the cat", "--max-tokens", 3, "--greedy")
    assert out.returncode == 0
    assert b"records no tokenizer fingerprint (it predates tokenizer v2); using the v2 tokenizer unverified" in out.stderr
    assert run(d / "m.bin", d / "t.tok").returncode == 2            # usage
    assert run(d / "m.bin", d / "t.tok", "x", "--top-p", 2).returncode == 2
    out = run(d / "missing.bin", d / "t.tok", "x")
    assert out.returncode == 1 and b"Could not open checkpoint for reading" in out.stderr


def test_bench_writes_the_reference_schema(tmp_path):
    """gradhip-bench: grad bench's generation section (src/cli/bench.cpp:269-286) and its JSON
    schema (:112-172)."""
    import json
    exe = os.path.join(ROOT, "grad.cpp_amd", "bin", "gradhip-bench")
    assert os.path.exists(exe), "gradhip-bench is not built; run __graft_entry__.build()"
    path = tmp_path / "bench.json"
    out = subprocess.run([exe, "--trials", "3", "--json", str(path)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "Generation throughput" in out.stdout and "median:" in out.stdout
    j = json.loads(path.read_text())
    assert list(j) == ["schema_version", "timestamp_utc", "engine", "version", "git_sha", "build_type", "compiler",
                       "system", "metal_available", "metal_fp16", "device", "parameters", "config", "protocol",
                       "training_steps_per_second", "training_tokens_per_second", "generation_tokens_per_second",
                       "median_training_steps_per_second", "median_training_tokens_per_second",
                       "median_generation_tokens_per_second", "peak_rss_mb", "metal_stream_per_step",
                       "metal_peak_live_mb"]
    assert j["schema_version"] == 1 and j["config"]["vocab"] == 5000 and j["config"]["d_model"] == 512
    # E, P, 6 x (4 d^2 + 4 d + 8 d^2 + 5 d + 4 d) and the final norm: the 22M configuration
    assert j["parameters"] == 5000 * 512 + 1024 * 512 + 6 * (12 * 512 * 512 + 13 * 512) + 2 * 512
    rates = j["generation_tokens_per_second"]
    assert len(rates) == 3 and all(r > 0 for r in rates)
    assert abs(j["median_generation_tokens_per_second"] - sorted(rates)[1]) < 1e-3
    assert subprocess.run([exe, "--trials", "0"], capture_output=True).returncode == 2


def test_chat_streams_each_line(setup):
    """gradhip-chat: `grad chat`'s loop (src/cli/chat.cpp:49-68): every line is encoded with a
    trailing newline, echoed, and continued token by token from an empty context."""
    d, tok, cfg, om = setup
    exe = os.path.join(ROOT, "grad.cpp_amd", "bin", "gradhip-chat")
    assert os.path.exists(exe), "gradhip-chat is not built; run __graft_entry__.build()"
    lines = ["the little cat", "Once upon a time"]
    out = subprocess.run([exe, str(d / "m.bin"), str(d / "t.tok"), "--max-tokens", "10", "--temperature", "0.9",
                          "--top-k", "8", "--repetition-penalty", "1.15", "--seed", "5"],
                         input=("\n".join(lines) + "\nexit\nnever read\n").encode(), capture_output=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    want = (b"\ngradhip Chat\n\n\nThis is a base language model: it continues text in the style of its training "
            b"corpus.\nEmpty line or 'exit' quits.\n\n")
    for line in lines:
        ids = tok.encode((line + "\n").encode())
        ref = O.generate_sample(om, ids, synth.uniforms(10, 5), 0.9, 10, 1.15, 8, 1.0)
        want += b"> " + line.encode() + tok.decode(ref[len(ids):]) + b"\n\n"
    want += b"> "
    assert out.stdout == want
    # --greedy is top-k 1: the arg-max stream without a draw mattering
    out = subprocess.run([exe, str(d / "m.bin"), str(d / "t.tok"), "--max-tokens", "6", "--greedy",
                          "--repetition-penalty", "1.0"], input=b"the cat\n\n", capture_output=True, timeout=120)
    ids = tok.encode(b"the cat\n")
    greedy = O.generate_greedy(om, ids, 6, 1.0)
    assert out.returncode == 0 and b"> the cat" + tok.decode(greedy[len(ids):]) + b"\n\n> " in out.stdout
    # --stop-at-eos: the reply ends after the tokenizer's end-of-text id; the stream up to there is
    # the reference's (which has no stop condition and runs on)
    eos = tok.vocab_size - 1  # the one special token comes last
    out = subprocess.run([exe, str(d / "m.bin"), str(d / "t.tok"), "--max-tokens", "40", "--temperature", "1.5",
                          "--seed", "61", "--stop-at-eos"], input=b"a dog\n\n", capture_output=True, timeout=120)
    ids = tok.encode(b"a dog\n")
    ref = list(O.generate_sample(om, ids, synth.uniforms(40, 61), 1.5, 40, 1.2, 0, 1.0)[len(ids):])
    assert eos in ref[3:30]  # the seed was chosen for this
    ref = ref[:ref.index(eos) + 1]
    assert out.returncode == 0 and b"> a dog" + tok.decode(ref) + b"\n\n> " in out.stdout


def test_chat_can_keep_its_context(setup):
    """--keep-context (not in grad.cpp, which starts every line from an empty context): a line is
    appended to the conversation so far, the draws go on where the last reply stopped, and a
    conversation that no longer fits starts over."""
    d, tok, cfg, om = setup
    exe = os.path.join(ROOT, "grad.cpp_amd", "bin", "gradhip-chat")
    lines = ["the little cat", "sat on", "the mat and the hat"]
    n = 25
    out = subprocess.run([exe, str(d / "m.bin"), str(d / "t.tok"), "--max-tokens", str(n), "--temperature", "0.9",
                          "--top-k", "8", "--repetition-penalty", "1.15", "--seed", "5", "--keep-context"],
                         input=("\n".join(lines) + "\n\n").encode(), capture_output=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    seed, drawn = 5, 0
    context, want, started_over = [], b"", 0
    for line in lines:
        ids = [int(t) for t in tok.encode((line + "\n").encode())]
        want += b"> " + line.encode()
        if len(context) + len(ids) >= cfg.max_len:
            want += b"\n[context full: starting over]"
            context, seed, drawn = [], seed + 1, 0  # a fresh session counts its draws from zero
            started_over += 1
        ref = O.generate_sample(om, context + ids, synth.uniforms(drawn + n, seed)[drawn:], 0.9, n, 1.15, 8, 1.0)
        want += tok.decode(ref[len(context) + len(ids):]) + b"\n\n"
        context = [int(t) for t in ref]
        drawn += n
    assert started_over == 1  # the third line does not fit the 64-token context
    assert out.stdout.endswith(want + b"> ")


def test_eval_scores_a_token_file(setup, tmp_path):
    """gradhip-eval: windows of a TOK1 file (src/data/token_file.cpp:149-176) in batches of eight,
    loss as training::mean_loss forms it (src/training/trainer.cpp:319-340)."""
    import re
    import struct

    import numpy as np
    d, tok, cfg, om = setup
    exe = os.path.join(ROOT, "grad.cpp_amd", "bin", "gradhip-eval")
    assert os.path.exists(exe), "gradhip-eval is not built; run __graft_entry__.build()"
    seq = 12
    tokens = synth.uniform_tokens(11 * seq + 5, cfg.vocab, 71)   # 11 windows: one full batch and one of three
    path = tmp_path / "val.bin"
    path.write_bytes(b"TOK1" + struct.pack("<IQ", cfg.vocab, len(tokens)) + tokens.astype("<u2").tobytes())
    out = subprocess.run([exe, str(d / "m.bin"), str(path), "--seq", str(seq)], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    m = re.search(r"^val\s+loss ([0-9.]+)  perplexity ([0-9.]+)  \((\d+) tokens, \d+s\)$", out.stdout, re.M)
    assert m, out.stdout
    windows = (len(tokens) - seq - 1) // seq + 1
    assert windows == 11 and int(m.group(3)) == windows * seq
    per_window = [O.score(om, tokens[w * seq:w * seq + seq], tokens[w * seq + 1:w * seq + seq + 1]).mean()
                  for w in range(windows)]
    batches = [per_window[:8], per_window[8:]]
    want = sum(np.mean(b) * len(b) for b in batches) / windows
    assert abs(float(m.group(1)) - want) <= 1e-3 and abs(float(m.group(2)) - np.exp(want)) <= 2e-3 * np.exp(want)
    # --batches 1: the first batch only
    out = subprocess.run([exe, str(d / "m.bin"), str(path), "--seq", str(seq), "--batches", "1"],
                         capture_output=True, text=True, timeout=120)
    m = re.search(r"loss ([0-9.]+)  perplexity [0-9.]+  \((\d+) tokens", out.stdout)
    assert out.returncode == 0 and int(m.group(2)) == 8 * seq and abs(float(m.group(1)) - np.mean(batches[0])) <= 1e-3
    # --sampled: windows drawn with replacement like grad.cpp's DataLoader under --max-batches; a few lines
    # of C++ built with the same library give the draws to expect
    draw = tmp_path / "draw.cpp"
    draw.write_text("#include <cstdio>\n#include <random>\nint main() { std::mt19937 g(20260921); "
                    "std::uniform_int_distribution<size_t> p(0, 10); "
                    "for (int i = 0; i < 11; i++) std::printf(\"%zu \", p(g)); }\n")
    subprocess.check_call(["g++", "-O1", str(draw), "-o", str(tmp_path / "draw")])
    drawn = [int(x) for x in subprocess.check_output([str(tmp_path / "draw")], text=True).split()]
    out = subprocess.run([exe, str(d / "m.bin"), str(path), "--seq", str(seq), "--batches", "2", "--sampled",
                          "--print-windows"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    listed = [[int(x) for x in line.split()[1:]] for line in out.stdout.split("\n") if line.startswith("windows")]
    assert listed == [drawn[:8], drawn[8:]] and len(set(drawn)) > 1
    want = sum(np.mean([per_window[w] for w in b]) * len(b) for b in listed) / 11
    m = re.search(r"loss ([0-9.]+)  perplexity [0-9.]+  \((\d+) tokens", out.stdout)
    assert int(m.group(2)) == 11 * seq and abs(float(m.group(1)) - want) <= 1e-3
    assert subprocess.run([exe, str(d / "m.bin"), str(path), "--sampled"], capture_output=True).returncode == 2
    # errors: a context longer than the model's, a file that is not a token file, the wrong vocabulary
    out = subprocess.run([exe, str(d / "m.bin"), str(path), "--seq", "65"], capture_output=True, text=True)
    assert out.returncode == 1 and "seq length exceeds the model's context (64)" in out.stderr
    out = subprocess.run([exe, str(d / "m.bin"), str(d / "t.tok"), "--seq", str(seq)], capture_output=True, text=True)
    assert out.returncode == 1 and "Not a token file (bad magic)" in out.stderr
    other = tmp_path / "other.bin"
    other.write_bytes(b"TOK1" + struct.pack("<IQ", cfg.vocab + 1, len(tokens)) + tokens.astype("<u2").tobytes())
    out = subprocess.run([exe, str(d / "m.bin"), str(other), "--seq", str(seq)], capture_output=True, text=True)
    assert out.returncode == 1 and "token files and checkpoint disagree on vocab size" in out.stderr
    assert subprocess.run([exe, str(d / "m.bin")], capture_output=True).returncode == 2


def test_generate_with_a_v1_tokenizer_cache(tmp_path):
    """A checkpoint trained with the v1 whitespace BPE (the reference's default for checkpoints
    that record no tokenizer, src/cli/common.cpp:160-187): same command, the cache file in
    place of the GTOK file."""
    v1 = R.train_v1(TEXT.replace("\n", " ").encode() * 3, 140)
    (tmp_path / "v1.cache").write_bytes(v1.cache_image())
    cfg = synth.Config(synth.ARCH_GPT2, v1.vocab_size, 128, 2, 2, 64)
    W = synth.make_weights(cfg, 33, std=lively_std(cfg), norm_noise=0.1)
    synth.write_checkpoint(str(tmp_path / "m.bin"), cfg, W, fingerprint=(1, v1.fingerprint()))
    om = O.Model.from_tensors(cfg, W)
    prompt = "Once upon a time,  the little cat"
    out = run(tmp_path / "m.bin", tmp_path / "v1.cache", prompt, "--max-tokens", 10, "--repetition-penalty", 1.2,
              "--greedy")
    assert out.returncode == 0, out.stdout + out.stderr
    ids = v1.encode(prompt.encode())
    greedy = O.generate_greedy(om, ids, 10, 1.2)
    assert f"Tokenizer: {tmp_path / 'v1.cache'} (v1, vocab {v1.vocab_size})\n".encode() in out.stdout
    assert b"--- Greedy Decoding ---\n\n" + f'Prompt: "{prompt}"\n'.encode() + v1.decode(greedy) + b"\n" in out.stdout
    # the same checkpoint refuses another v1 vocabulary of the same size
    vocab = sorted(v1.vocab.items(), key=lambda kv: kv[1])
    other = R.BpeV1Ref(vocab[:-1] + [(b"\x7f\x7f", vocab[-1][1])], v1.merges[:-1])
    assert other.vocab_size == v1.vocab_size and other.fingerprint() != v1.fingerprint()
    (tmp_path / "other.cache").write_bytes(other.cache_image())
    out = run(tmp_path / "m.bin", tmp_path / "other.cache", prompt, "--greedy")
    assert out.returncode == 1
    assert (f"Error: tokenizer v1:{other.fingerprint():016x} is not the one {tmp_path / 'm.bin'} was trained with "
            f"(v1:{v1.fingerprint():016x})").encode() in out.stderr


def test_generate_finds_the_tokenizer_from_the_corpus_path(setup, tmp_path):
    """`grad generate <checkpoint> <prompt> [corpus]` names no tokenizer file: it follows from the
    corpus path, the checkpoint's vocabulary and its recorded tokenizer generation
    (src/cli/common.cpp:346-358).  The same call shape here, with --corpus."""
    d, tok, cfg, om = setup
    corpus = tmp_path / "stories.txt"
    corpus.write_text(TEXT)
    tok_file = f"{corpus}.bytebpe_{tok.vocab_size}.tok"
    open(tok_file, "wb").write(tok.file_image())
    prompt = "the little cat"
    out = run(d / "m.bin", prompt, "--corpus", corpus, "--max-tokens", 8, "--repetition-penalty", 1.1, "--greedy")
    assert out.returncode == 0, out.stdout + out.stderr
    greedy = O.generate_greedy(om, tok.encode(prompt.encode()), 8, 1.1)
    assert f"Tokenizer: {tok_file} (v2, vocab {tok.vocab_size})\n".encode() in out.stdout
    assert tok.decode(greedy) + b"\n" in out.stdout
    # the flag may not contradict the checkpoint; a checkpoint without a record means v1, whose cache is not there
    out = run(d / "m.bin", prompt, "--corpus", corpus, "--tokenizer", "v1", "--greedy")
    assert out.returncode == 1
    assert b"--tokenizer v1 does not match the checkpoint, which was trained with tokenizer v2:" in out.stderr
    out = run(d / "plain.bin", prompt, "--corpus", corpus, "--greedy")
    assert out.returncode == 1
    assert (f"Error: No v1 tokenizer {corpus}.tokenizer_{tok.vocab_size}.cache; run: ./build/grad prepare {corpus} "
            f"{tok.vocab_size} --tokenizer v1").encode() in out.stderr
    out = run(d / "plain.bin", prompt, "--corpus", corpus, "--tokenizer", "v2", "--max-tokens", 3, "--greedy")
    assert out.returncode == 0 and b"using the v2 tokenizer unverified" in out.stderr
    assert run(d / "m.bin", prompt, "--corpus", corpus, "--tokenizer", "v3").returncode == 2
    assert run(d / "m.bin", d / "t.tok", prompt, "--tokenizer", "v2").returncode == 2   # the flag needs --corpus
