"""Pins the checkpoint reader/writer (oracle AND product host code) to the facts
grad.cpp's own test asserts: tests/unit/test_core_regressions.cpp:426-541."""
import os
import struct

import numpy as np
import pytest

import gradhip as G
import oracle_lib as O
from gradhip import synth

ARCHS = [synth.ARCH_GPT2, synth.ARCH_MODERN]


def _good(tmp_path, arch, fingerprint=None):
    # The reference test's shape: vocab 11, d 8, 2 layers, 2 heads, max_len 6.
    cfg = synth.Config(arch, 11, 8, 2, 2, 6)
    W = synth.make_weights(cfg, 42, std=0.3, norm_noise=0.1)
    path = str(tmp_path / f"model{arch}.bin")
    synth.write_checkpoint(path, cfg, W, fingerprint)
    return cfg, W, path


def _oracle_fails(path):
    with pytest.raises(RuntimeError) as e:
        O.Model.load(path)
    return str(e.value)


def _product_fails(path):
    # The product validates the file on the host before it touches the GPU, so
    # these messages are checkable without one.
    with pytest.raises(RuntimeError) as e:
        G.Model.load(path)
    return str(e.value)


FAILS = [_oracle_fails, _product_fails]


@pytest.mark.parametrize("arch", ARCHS)
def test_oracle_round_trip_is_bitwise(tmp_path, arch):
    cfg, W, path = _good(tmp_path, arch)
    m = O.Model.load(path)
    assert m.num_tensors == len(W)
    for i, w in enumerate(W):
        assert np.array_equal(m.tensor(i).view(np.uint32), w.view(np.uint32))
    again = str(tmp_path / "again.bin")
    m.save(again)
    assert open(again, "rb").read() == open(path, "rb").read()
    d = m.dims()
    assert (d["vocab"], d["d_model"], d["layers"], d["heads"], d["max_len"]) == (11, 8, 2, 2, 6)
    assert d["d_ff"] == (64 if arch == synth.ARCH_MODERN else 32)


@pytest.mark.parametrize("arch", ARCHS)
def test_header_byte_offsets(tmp_path, arch):
    # test_core_regressions.cpp:455-457: magic@0, version@4, arch@8, vocab@12, d_model@16,
    # layers@20, heads@24, max_len@28, dropout@32, first tensor rows@36.
    _, _, path = _good(tmp_path, arch)
    b = open(path, "rb").read()
    assert len(b) > 64
    assert b[:4] == b"MTPG"  # 0x4750544D little-endian
    assert struct.unpack_from("<IIIiiiiif", b, 0) == (0x4750544D, 2, arch, 11, 8, 2, 2, 6, 0.0)
    assert struct.unpack_from("<ii", b, 36) == (11, 8)


@pytest.mark.parametrize("fails", FAILS)
@pytest.mark.parametrize("arch", ARCHS)
def test_rejections_carry_the_reference_messages(tmp_path, arch, fails):
    _, _, path = _good(tmp_path, arch)
    good = open(path, "rb").read()
    bad = str(tmp_path / "bad.bin")

    def write(data):
        open(bad, "wb").write(data)

    def poke(fmt, off, val):
        b = bytearray(good)
        struct.pack_into(fmt, b, off, val)
        return bytes(b)

    write(good[:-10])
    assert "file ends inside final norm beta" in fails(bad)
    write(good[:20])
    assert "file ends while reading num_layers" in fails(bad)
    write(poke("<I", 8, 7))
    assert "unknown architecture tag 7" in fails(bad)
    write(poke("<i", 16, -5))
    assert "d_model = -5" in fails(bad)
    write(poke("<i", 24, 3))
    assert "not divisible" in fails(bad)
    write(poke("<i", 36, 12))
    msg = fails(bad)
    assert "token embedding is 12x8, model expects 11x8" in msg
    assert bad in msg  # the path is in every message
    assert msg.startswith("Failed to load model from " + bad + ": ")
    # further header rules of GPTModel::load (gpt_model.cpp:391-430)
    write(poke("<I", 0, 0x12345678))
    assert "not a grad.cpp checkpoint (wrong magic number)" in fails(bad)
    write(poke("<I", 4, 3))
    assert "unsupported format version 3" in fails(bad)
    write(poke("<i", 12, 0))
    assert "header field vocab_size = 0 is outside [1, 16777216]" in fails(bad)
    write(poke("<i", 28, (1 << 20) + 1))
    assert "header field max_len = 1048577 is outside [1, 1048576]" in fails(bad)
    write(poke("<f", 32, 1.0))
    assert "dropout_rate 1.000000 is outside [0, 1)" in fails(bad)
    write(good[:2])
    assert "file ends while reading magic number" in fails(bad)
    assert "Could not open checkpoint for reading: " in fails(str(tmp_path / "missing.bin"))


@pytest.mark.parametrize("fails", FAILS)
@pytest.mark.parametrize("arch", ARCHS)
def test_tokenizer_trailer(tmp_path, arch, fails):
    cfg, W, path = _good(tmp_path, arch)
    good = open(path, "rb").read()
    fp = (2, 0x0123456789ABCDEF)
    tagged_path = str(tmp_path / "tagged.bin")
    synth.write_checkpoint(tagged_path, cfg, W, fp)
    tagged = open(tagged_path, "rb").read()
    # +20 bytes after an unchanged prefix (test_core_regressions.cpp:495-504)
    assert len(tagged) == len(good) + 20 and tagged[:len(good)] == good
    assert O.Model.load(path).fingerprint() is None
    m = O.Model.load(tagged_path)
    assert m.fingerprint() == fp
    resaved = str(tmp_path / "resaved.bin")
    m.save(resaved)
    assert open(resaved, "rb").read() == tagged

    bad = str(tmp_path / "bad.bin")
    # Unknown sections are skipped (:506-517).
    open(bad, "wb").write(good + b"ZZZZ\x03\x00\x00\x00abc" + tagged[len(good):])
    assert O.Model.load(bad).fingerprint() == fp
    # Corrupt trailers (:519-538).
    open(bad, "wb").write(tagged[:-3])
    assert "file ends while reading tokenizer trailer" in fails(bad)
    open(bad, "wb").write(tagged[:len(good) + 3])
    assert "file ends while reading trailer section header" in fails(bad)
    b = bytearray(tagged)
    struct.pack_into("<I", b, len(good) + 8, 9)
    open(bad, "wb").write(bytes(b))
    assert "unknown tokenizer kind 9" in fails(bad)
    b = bytearray(tagged)
    struct.pack_into("<I", b, len(good) + 4, 11)
    open(bad, "wb").write(bytes(b))
    assert "tokenizer trailer has length 11" in fails(bad)
    b = bytearray(tagged)
    struct.pack_into("<I", b, len(good) + 4, 0x7FFFFFFF)
    open(bad, "wb").write(bytes(b))
    assert "implausible length" in fails(bad)
    open(bad, "wb").write(good + b"ZZZZ\x10\x00\x00\x00abc")
    assert "file ends inside trailer section" in fails(bad)


def test_v1_files_load_as_gpt2(tmp_path):
    # gpt_model.cpp:399-409: version 1 has no arch tag and is always GPT-2.
    cfg = synth.Config(synth.ARCH_GPT2, 11, 8, 2, 2, 6)
    W = synth.make_weights(cfg, 3)
    path = str(tmp_path / "v1.bin")
    synth.write_checkpoint(path, cfg, W, version=1)
    assert struct.unpack_from("<i", open(path, "rb").read(), 8)[0] == 11  # vocab sits where arch would
    m = O.Model.load(path)
    assert m.dims()["arch"] == synth.ARCH_GPT2
    assert np.array_equal(m.tensor(0), W[0])


@pytest.mark.parametrize("fails", FAILS)
def test_modern_needs_an_even_head_size(tmp_path, fails):
    # load() constructs the model, whose attention rejects an odd head size
    # under RoPE (multihead_attention.cpp:333-335).
    path = str(tmp_path / "odd.bin")
    with open(path, "wb") as f:
        f.write(struct.pack("<III5if", 0x4750544D, 2, 1, 11, 9, 1, 3, 6, 0.0))
    assert "RoPE requires an even head size" in fails(path)
