"""Builds libgradhip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
from __future__ import annotations

import os
import subprocess
import sys

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB = os.path.join(LIB_DIR, "libgradhip.so")

# -packed-fp32-ops is switched off on purpose: some packed fp32 forms have given
# wrong results on this hardware pool.  No fast-math: GELU/SiLU/softmax/RoPE use
# the precise expf/tanhf.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-fast-math", "-Wall", "-Wno-unused-function", *os.environ.get("GRADHIP_EXTRA_FLAGS", "").split(),
]
SOURCES = ["engine.hip", "checkpoint.cpp", "tokenizer.cpp"]


BIN_DIR = os.path.join(PKG, "bin")
CLI = os.path.join(BIN_DIR, "gradhip-generate")
INCLUDE = os.path.join(os.path.dirname(PKG), "include")


def build(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, "-o", LIB, *[os.path.join(CSRC, s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # the command-line caller: plain C++ over the header-only adapter
    os.makedirs(BIN_DIR, exist_ok=True)
    for src, exe in (("generate.cpp", CLI), ("chat.cpp", os.path.join(BIN_DIR, "gradhip-chat")),
                     ("bench.cpp", os.path.join(BIN_DIR, "gradhip-bench")),
                     ("eval.cpp", os.path.join(BIN_DIR, "gradhip-eval"))):
        cmd = ["g++", "-std=c++20", "-O2", "-Wall", "-Wextra", "-I", INCLUDE, os.path.join(PKG, "cli", src),
               "-o", exe, "-L", LIB_DIR, "-lgradhip", "-Wl,-rpath,$ORIGIN/../lib"]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
