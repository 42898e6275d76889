"""Logits of a few sequences against a large vocabulary: the projection whose weight
matrix (vocab x d_model) is far wider than the batch is deep takes a kernel of its
own (rows of the batch held in registers, weight tiles streamed past them).  Every
shape it is compiled for - d_model 512, 768, 1024; up to 16 and up to 32 rows; both
block families (RMSNorm folded into the projection, LayerNorm ahead of it) - and a
vocabulary that ends inside a tile and inside a workgroup's run of tiles, must give
the logits of InferenceSession::step (inference.cpp:251-257) per sequence; batches
just past its range (33 rows) take the general tiles and are checked beside it."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import assert_logits_close, make_pair

pytestmark = pytest.mark.gpu

# (arch, vocab, d_model, heads): one layer, context 6
SHAPES = {
    "modern-d768": (synth.ARCH_MODERN, 8207, 768, 12),
    "gpt2-d768": (synth.ARCH_GPT2, 8207, 768, 12),
    "modern-d512": (synth.ARCH_MODERN, 8193, 512, 8),
    "gpt2-d1024": (synth.ARCH_GPT2, 8250, 1024, 16),
    "modern-d1024": (synth.ARCH_MODERN, 8272, 1024, 16),
}


@pytest.fixture(scope="module")
def pairs():
    O.blas_init()
    out = {}
    for name, (arch, vocab, d, heads) in SHAPES.items():
        cfg = synth.Config(arch, vocab, d, 1, heads, 6)
        W, om = make_pair(cfg, 77, std=0.05, norm_noise=0.1)
        out[name] = (cfg, om, G.Model.from_tensors(cfg, W))
    return out


@pytest.mark.parametrize("name", sorted(SHAPES))
@pytest.mark.parametrize("batch", [2, 16, 17, 32, 33])
def test_step_logits_per_sequence(pairs, name, batch):
    cfg, om, gm = pairs[name]
    gs = G.Session(gm, batch=batch)
    toks = synth.uniform_tokens(batch * 3, cfg.vocab, 500 + batch).reshape(batch, 3)
    # the oracle walks three sequences of the batch: the first, one in the middle, the last
    watch = sorted({0, batch // 2, batch - 1})
    oss = {b: O.Session(om) for b in watch}
    for t in range(3):
        got = gs.step(toks[:, t])
        assert got.shape == (batch, cfg.vocab)
        for b in watch:
            assert_logits_close(got[b], oss[b].step(int(toks[b, t])), what=f"{name} B={batch} seq {b} step {t}")
    assert gs.position == 3
