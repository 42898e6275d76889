"""Which tokenizer file belongs to a checkpoint: the naming and choice rules of grad.cpp's
commands (src/cli/common.cpp:101-124 names, :160-187 choose_tokenizer, :43-59 and :236-252
loading), as `grad.cpp_amd/cli/resolve.h` restates them.  A C++ driver compiled with g++
prints what the rules give for a directory of prepared files; needs no GPU."""
import os
import subprocess
import sys

from gradhip import LIB_PATH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import tokenizer_ref as R  # noqa: E402


def test_tokenizer_resolution_rules(tmp_path):
    exe = str(tmp_path / "resolve_test")
    lib_dir = os.path.dirname(LIB_PATH)
    subprocess.check_call(["g++", "-std=c++20", "-O1", "-Wall", "-Wextra", "-I", os.path.join(ROOT, "include"),
                           "-I", os.path.join(ROOT, "grad.cpp_amd", "cli"),
                           os.path.join(ROOT, "tests", "cpp", "resolve_test.cpp"), "-o", exe,
                           "-L", lib_dir, "-lgradhip", f"-Wl,-rpath,{lib_dir}"])
    text = "the cat sat on the mat and the cat ran to the hat\n" * 8
    v2 = R.train(text.encode(), 300)
    v1 = R.train_v1(text.replace("\n", " ").encode(), 60)
    d = tmp_path / "corpus"
    d.mkdir()
    c = str(d / "c.txt")
    (d / "c.txt").write_text(text)
    open(f"{c}.bytebpe_300.tok", "wb").write(v2.file_image())        # 300: v2 file
    open(f"{c}.tokenizer_301.cache", "wb").write(v1.cache_image())   # 301: v1 cache
    open(f"{c}.bytebpe_302.tok", "wb").write(v2.file_image())        # 302: both
    open(f"{c}.tokenizer_302.cache", "wb").write(v1.cache_image())
    for split in ("train", "val"):                                   # 304: prepared for v1, no cache file
        open(f"{c}.304.{split}.bin", "wb").write(b"\0" * 8)
    open(f"{c}.v2.305.train.bin", "wb").write(b"\0" * 8)             # 305: half prepared for v2: does not count
    open(f"{c}.bytebpe_306.tok", "wb").write(v1.cache_image())       # 306: a v1 cache under a v2 name
    out = subprocess.run([exe, str(d), "c.txt"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    got = dict(line.split(" ", 1) for line in out.stdout.strip().split("\n") if not line.startswith("Tokenizer: "))
    assert got["v2"] == "data/c.txt.bytebpe_8000.tok"
    assert got["v1"] == "data/c.txt.tokenizer_8000.cache"
    assert got["v1-default"] == "tokenizer_5000.cache"            # the default corpus keeps its old cache name
    assert got["v2-default"] == "data/shakespeare.txt.bytebpe_5000.tok"
    assert got["bin-v1"] == "data/c.txt.8000.train.bin"
    assert got["bin-v2"] == "data/c.txt.v2.8000.val.bin"
    assert got["flag-v1"] == "v1" and got["flag-v2"] == "v2" and got["flag-none"] == "unset"
    assert got["flag-bad"] == "usage: --tokenizer: expected v1 or v2, got 'v3'"
    assert got["ckpt-recorded-v2"] == "v2" and got["ckpt-recorded-v2-asked-v2"] == "v2"
    assert got["ckpt-recorded-v2-asked-v1"] == ("error: --tokenizer v1 does not match the checkpoint, which was "
                                                "trained with tokenizer v2:1122334455667788")
    assert got["ckpt-recorded-v1"] == "v1"
    assert got["ckpt-unrecorded"] == "v1"              # a checkpoint without a fingerprint predates v2
    assert got["ckpt-unrecorded-asked-v2"] == "v2"
    assert got["files-300"] == "v2" and got["files-301"] == "v1"
    assert got["files-302"] == (f"error: both a v1 tokenizer ({c}.tokenizer_302.cache) and a v2 tokenizer "
                                f"({c}.bytebpe_302.tok) exist for {c} at vocab 302; pass --tokenizer v1 or "
                                "--tokenizer v2")
    assert got["files-302-asked-v1"] == "v1"
    assert got["files-303"] == "v2"                    # nothing on disk: the current generation
    assert got["files-304"] == "v1" and got["files-305"] == "v2"
    assert got["load-v2"] == str(v2.vocab_size) and got["load-v1"] == str(v1.vocab_size)
    assert f"Tokenizer: {c}.bytebpe_300.tok (v2, vocab {v2.vocab_size})" in out.stdout
    assert got["load-missing"] == (f"error: No v2 tokenizer {c}.bytebpe_303.tok; run: ./build/grad prepare {c} 303 "
                                   "--tokenizer v2")
    assert got["load-wrong-kind"].startswith("error: ")
    assert got["vocab-mismatch"] == (f"error: tokenizer has {v2.vocab_size} tokens but the checkpoint expects 999; "
                                     "the cache was built for a different vocab or corpus")
