"""The committed fixture tests/golden/forward_float64.npz (rows of the full
forward in float64 for the reference's parity-test shapes and sequence,
sanity_tests.cpp:293-333) against the CPU oracle and, on a GPU, against the HIP
path: step(i) must reproduce row i."""
import os

import numpy as np
import pytest

import oracle_lib as O
from gradhip import synth
from helpers import TINY_SHAPES, assert_logits_close, lively_std

GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "forward_float64.npz"))
NAMES = [k for k in GOLDEN.files if k in TINY_SHAPES]


def weights(name):
    cfg = TINY_SHAPES[name]
    return cfg, synth.make_weights(cfg, int(GOLDEN["seed"]), std=lively_std(cfg), norm_noise=0.1)


def test_fixture_covers_the_reference_shapes():
    assert {"ref-sanity-gpt2", "ref-sanity-modern", "ref-metal-gpt2", "ref-metal-modern"} <= set(NAMES)
    assert GOLDEN["sequence"].tolist() == [3, 11, 7, 0, 19, 5]  # sanity_tests.cpp:301


@pytest.mark.parametrize("name", NAMES)
def test_oracle_steps_reproduce_the_golden_rows(name):
    cfg, W = weights(name)
    sess = O.Session(O.Model.from_tensors(cfg, W))
    for i, tok in enumerate(GOLDEN["sequence"]):
        assert_logits_close(sess.step(int(tok)), GOLDEN[name][i], 1e-4, f"{name} row {i}")


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("name", NAMES)
def test_gpu_steps_reproduce_the_golden_rows(name, batch):
    import gradhip as G
    cfg, W = weights(name)
    gm = G.Model.from_tensors(cfg, W)
    engines = [G.ENGINE_GRAPH, G.ENGINE_EAGER] if batch == 1 else [G.ENGINE_GRAPH]
    for engine in engines:
        s = G.Session(gm, batch=batch, engine=engine)
        for i, tok in enumerate(GOLDEN["sequence"]):
            logits = s.step([int(tok)] * batch)
            for b in range(batch):
                assert_logits_close(logits[b], GOLDEN[name][i], 1e-4, f"{name} row {i} seq {b} engine {engine}")
    # the whole sequence in one prompt pass ends on the last row
    s = G.Session(gm, batch=batch)
    last = s.prefill(np.tile(GOLDEN["sequence"], (batch, 1)))
    for b in range(batch):
        assert_logits_close(last[b], GOLDEN[name][-1], 1e-4, f"{name} prompt pass seq {b}")
