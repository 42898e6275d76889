"""Writes tests/golden/forward_float64.npz: logits of the full-sequence forward for
the reference's own parity-test shapes and token sequence, from the float64
restatement of GPTModel::forward in tests/ref_forward.py.

The reference pins step() by exactly this invariant: the logits of step(i) equal
row i of the full forward (tests/integration/sanity_tests.cpp:293-333, sequence
at :301, shapes at :296-299 and tests/integration/metal_parity.cpp:345-352).  The
reference binary cannot be built in this image, so the expected rows come from an
independent restatement in float64 instead of from the binary; weights are the
seeded synthetic ones of gradhip.synth (Philox4x32-10 + Box-Muller), which every
consumer of the fixture regenerates from the seed.

Run from the repository root:  python tests/golden/make_forward_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path[:0] = [os.path.join(ROOT, "grad.cpp_amd"), os.path.join(ROOT, "tests")]

import ref_forward as R  # noqa: E402
from gradhip import synth  # noqa: E402
from helpers import REF_SEQUENCE, TINY_SHAPES, lively_std  # noqa: E402

SEED = 4242
NAMES = ["ref-sanity-gpt2", "ref-sanity-modern", "ref-metal-gpt2", "ref-metal-modern", "hs64-gpt2", "hs64-modern"]


def main():
    out = {"sequence": np.asarray(REF_SEQUENCE, dtype=np.int32), "seed": np.int64(SEED)}
    for name in NAMES:
        cfg = TINY_SHAPES[name]
        W = synth.make_weights(cfg, SEED, std=lively_std(cfg), norm_noise=0.1)
        logits = R.forward(cfg, W, REF_SEQUENCE)
        out[name] = logits.astype(np.float32)
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "forward_float64.npz"), **out)
    print({k: getattr(v, "shape", v) for k, v in out.items()})


if __name__ == "__main__":
    main()
