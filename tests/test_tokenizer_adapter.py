"""The tokenizer classes of the header-only C++ adapter (include/gradhip.hpp), driven
by a C++ caller compiled with g++ against the C ABI.  Needs no GPU."""
import os
import subprocess
import sys

from gradhip import LIB_PATH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import tokenizer_ref as R  # noqa: E402


def test_cpp_tokenizer_caller_matches_the_oracle(tmp_path):
    exe = str(tmp_path / "tokenizer_adapter_test")
    lib_dir = os.path.dirname(LIB_PATH)
    subprocess.check_call(["g++", "-std=c++20", "-O1", "-Wall", "-Wextra", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "cpp", "tokenizer_adapter_test.cpp"), "-o", exe,
                           "-L", lib_dir, "-lgradhip", f"-Wl,-rpath,{lib_dir}"])
    text = "Once upon a time, the little cat said: don't go!\n<|endoftext|>The end  "
    ref = R.train((text * 3 + "the cat sat on the mat and the cat ran to the hat\n" * 5).encode(), 330)
    path = tmp_path / "t.tok"
    path.write_bytes(ref.file_image())
    v1 = R.train_v1(text.replace("\n", " ").encode() * 3, 120)
    v1_path = tmp_path / "v1.cache"
    v1_path.write_bytes(v1.cache_image())
    one_line = "Once upon a time,   the little_cat said"
    out = subprocess.run([exe, str(path), one_line, str(v1_path)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    lines = out.stdout.strip().split("\n")
    assert lines[9] == f"v1 v1:{v1.fingerprint():016x} vocab {v1.vocab_size} eos 1 unk 2"
    assert [int(x) for x in lines[10].split()[1:]] == v1.encode(one_line.encode())
    assert lines[11] == "v1text Once upon a time, the little cat said"
    assert lines[12] == f"runtime_error Tokenizer file {v1_path}: not a GTOK tokenizer file"
    out = subprocess.run([exe, str(path), text], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    lines = out.stdout.strip().split("\n")
    eos = 256 + len(ref.merges)
    assert lines[0] == f"kind v2 vocab {ref.vocab_size} eos {eos}"
    assert lines[1] == f"identity v2:{ref.fingerprint():016x}"
    assert [int(x) for x in lines[2].split()[1:]] == ref.encode(text.encode())
    assert eos in ref.encode(text.encode())
    assert lines[3] == "round_trip 1"
    assert lines[4] == f"special {eos} 0"
    assert lines[5] == f"out_of_range token id {ref.vocab_size} is outside the vocabulary of {ref.vocab_size}"
    assert lines[6] == "runtime_error Failed to open tokenizer file: /nonexistent/tok.tok"
    assert lines[7] == "invalid_argument merge 1 repeats an earlier merge"
    assert lines[8] == "tiny v2:08b0b6b208dca2a9"  # the value grad.cpp's test freezes
