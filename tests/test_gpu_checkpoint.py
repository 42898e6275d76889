"""GPU side of the checkpoint contract: files load onto the device, and
gh_model_save reads the weights back into a byte-identical file
(tests/unit/test_core_regressions.cpp:438-452 asks for a bitwise round trip)."""
import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth
from helpers import assert_logits_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("arch", [synth.ARCH_GPT2, synth.ARCH_MODERN])
@pytest.mark.parametrize("fingerprint", [None, (2, 0x0123456789ABCDEF), (1, 0xBA36BE291B13AD8E)])
def test_load_save_round_trip_is_bitwise(tmp_path, arch, fingerprint):
    cfg = synth.Config(arch, 211, 64, 2, 4, 24)
    W = synth.make_weights(cfg, 5, std=0.1, norm_noise=0.1)
    src, dst = str(tmp_path / "a.bin"), str(tmp_path / "b.bin")
    synth.write_checkpoint(src, cfg, W, fingerprint)
    m = G.Model.load(src)
    c = m.config
    assert (c.arch, c.vocab, c.d_model, c.layers, c.heads, c.max_len) == (arch, 211, 64, 2, 4, 24)
    assert c.d_ff == cfg.d_ff
    assert bool(c.has_fingerprint) == (fingerprint is not None)
    if fingerprint:
        assert (c.tokenizer_kind, c.tokenizer_hash) == fingerprint
    m.save(dst)
    assert open(src, "rb").read() == open(dst, "rb").read()
    # and the oracle reads the product's file
    om = O.Model.load(dst)
    assert om.fingerprint() == fingerprint


def test_loaded_file_decodes_like_the_oracle(tmp_path):
    cfg = synth.Config(synth.ARCH_MODERN, 211, 64, 2, 4, 24)
    W = synth.make_weights(cfg, 6, std=0.14, norm_noise=0.1)
    path = str(tmp_path / "m.bin")
    synth.write_checkpoint(path, cfg, W)
    gs, osess = G.Session(G.Model.load(path)), O.Session(O.Model.load(path))
    for t in synth.uniform_tokens(24, 211, 1):
        assert_logits_close(gs.step([t])[0], osess.step(t), 1e-4)


def test_v1_file_loads_as_gpt2(tmp_path):
    cfg = synth.Config(synth.ARCH_GPT2, 50, 16, 1, 2, 8)
    W = synth.make_weights(cfg, 7, std=0.2)
    path = str(tmp_path / "v1.bin")
    synth.write_checkpoint(path, cfg, W, version=1)
    m = G.Model.load(path)
    assert m.config.arch == synth.ARCH_GPT2
    gs, osess = G.Session(m), O.Session(O.Model.from_tensors(cfg, W))
    assert_logits_close(gs.step([3])[0], osess.step(3), 1e-4)


def test_save_to_missing_directory_fails(tmp_path):
    cfg = synth.Config(synth.ARCH_GPT2, 50, 16, 1, 2, 8)
    m = G.Model.from_tensors(cfg, synth.make_weights(cfg, 7))
    with pytest.raises(RuntimeError, match="Could not open file for writing"):
        m.save(str(tmp_path / "no_such_dir" / "x.bin"))


def test_from_host_validates_like_the_loader():
    with pytest.raises(RuntimeError, match="not divisible"):
        G.Model.from_tensors(synth.Config(synth.ARCH_GPT2, 50, 16, 1, 3, 8), [np.zeros((1, 1), np.float32)])
    cfg = synth.Config(synth.ARCH_GPT2, 50, 16, 1, 2, 8)
    with pytest.raises(ValueError, match="tensor count"):
        G.Model.from_tensors(cfg, synth.make_weights(cfg, 1)[:-1])
