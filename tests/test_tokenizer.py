"""The byte-level BPE tokenizer of the library (host code behind the C ABI) against
(1) the known answers grad.cpp's own tests hold (tests/golden/tokenizer_cases.json) and
(2) the CPU restatement in oracle/tokenizer_ref.py, which is itself pinned by the same
known answers first.  Needs no GPU: the tokenizer runs on the host in grad.cpp too."""
import json
import os
import random

import numpy as np
import pytest

import gradhip as G

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
import sys

sys.path.insert(0, os.path.join(ROOT, "oracle"))
import tokenizer_ref as R  # noqa: E402

CASES = json.load(open(os.path.join(ROOT, "tests", "golden", "tokenizer_cases.json")))
H = bytes.fromhex
EOT = b"<|endoftext|>"


def corpus(seed, words):
    """Plain English-like text with punctuation, digits, blank lines and some non-ASCII."""
    rng = random.Random(seed)
    vocab = ("the cat sat on a mat and she said hello to little girl who loved play day once upon time "
             "there was big red ball it's don't we'll 42 2024 3.14 café naïve 日本語 "
             "\U0001F600 e-mail __init__ x²").split()
    syllables = "ka to mi ra ne lo shi an der wol fen bur qui zet pla".split()
    out = []
    for i in range(words):
        if rng.random() < 0.3:  # made-up words keep the pair statistics rich
            out.append("".join(rng.choice(syllables) for _ in range(rng.randrange(1, 5))))
        else:
            out.append(rng.choice(vocab))
        r = rng.random()
        out.append(" " if r < 0.8 else ".\n" if r < 0.9 else ", " if r < 0.95 else "\n\n  ")
    return "".join(out).encode()


def random_bytes(rng, n):
    return bytes(rng.randrange(256) for _ in range(n))


@pytest.fixture(scope="module")
def trained():
    ref = R.train(corpus(1, 4000), 700)
    assert ref.vocab_size == 700
    return ref, G.Tokenizer.from_merges(ref.merges, ref.specials)


# ---------------------------------------------------------------- the oracle, pinned

def test_oracle_fnv1a_published_vectors():
    assert R.fnv1a64(b"") == 0xcbf29ce484222325
    assert R.fnv1a64(b"a") == 0xaf63dc4c8601ec8c
    assert R.fnv1a64(b"foobar") == 0x85944171f73967e8


def test_oracle_split_matches_golden():
    for c in CASES["splits"]:
        assert R.split(H(c["text"])) == [H(p) for p in c["pieces"]], c


def test_oracle_frozen_fingerprint():
    for f in CASES["frozen_fingerprints"]:
        tok = R.ByteBpeRef([tuple(m) for m in f["merges"]], [H(s) for s in f["specials"]])
        assert f"{tok.fingerprint():016x}" == f["fingerprint"]


def test_oracle_training_tie_breaks():
    for c in CASES["tie_breaks"]:
        got = R.train(H(c["text"]), c["vocab"], [H(s) for s in c["specials"]]).merges
        assert got == [tuple(m) for m in c["merges"]], c
    assert R.train(b"abc", 1000, []).vocab_size == 258  # stops when the pairs run out


def test_oracle_overlapping_specials():
    o = CASES["overlapping_specials"]
    tok = R.ByteBpeRef([], [H(s) for s in o["specials"]])
    for c in o["cases"]:
        assert tok.encode(H(c["text"])) == [256 + int(i[1:]) for i in c["ids"]]


def test_oracle_file_round_trip():
    ref = R.train(corpus(4, 500), 300)
    again = R.parse_file(ref.file_image())
    assert (again.merges, again.specials) == (ref.merges, ref.specials)
    assert len(ref.file_image()) == 24 + 8 + len(EOT) + 8 * len(ref.merges) + 8


# ---------------------------------------------------------------- pre-tokenizer

def test_golden_splits():
    for c in CASES["splits"]:
        assert G.pretokenize(H(c["text"])) == [H(p) for p in c["pieces"]], c


def test_character_classes():
    for c in CASES["classes"]:
        assert G.codepoint_class(c["codepoint"]) == c["class"], hex(c["codepoint"])
    assert G.codepoint_class(0x110000) == 0


def test_every_codepoint_class_matches_the_regex_module():
    """All 1,114,112 code points against the `regex` module, whose database is newer than the
    tokenizer's Unicode 16.0: the letters and digits added since are "other" here (their range
    ends are pinned by samples of grad.cpp's table in test_character_classes)."""
    import regex
    kinds = [regex.compile(p) for p in (r"\p{L}", r"\p{N}", r"\s")]
    newer = set()
    for lo, hi in R.AGE_17:
        newer.update(range(lo, hi + 1))
    lib = G.load_library()
    bad = []
    for cp in range(0x110000):
        ch = chr(cp)
        want = 3 if kinds[2].match(ch) else 1 if kinds[0].match(ch) else 2 if kinds[1].match(ch) else 0
        if cp in newer:
            assert want in (1, 2), hex(cp)
            want = 0
        if lib.gh_codepoint_class(cp) != want:
            bad.append(hex(cp))
    assert not bad, bad[:20]


def test_invalid_utf8_is_one_scalar_per_byte():
    for hx in CASES["invalid_utf8"]:
        b = H(hx)
        # an invalid byte is class "other": between two letters it stands alone
        pieces = G.pretokenize(b"a" + b + b"a")
        assert pieces[0] == b"a" and pieces[-1] == b"a" and b"".join(pieces[1:-1]) == b
        assert pieces == R.split(b"a" + b + b"a")
    # valid multi-byte sequences are one scalar: U+10FFFF (other), e acute (letter)
    assert G.pretokenize(b"a\xf4\x8f\xbf\xbfa") == [b"a", b"\xf4\x8f\xbf\xbf", b"a"]
    assert G.pretokenize(b"a\xc3\xa9a") == [b"a\xc3\xa9a"]


def test_splits_match_oracle_on_random_text():
    rng = random.Random(7)
    for trial in range(300):
        text = random_bytes(rng, rng.randrange(200))
        if trial % 2 == 0:
            text += corpus(rng.randrange(1 << 30), 20)
        if trial % 5 == 0:  # random valid code points, including astral ones
            text += "".join(chr(rng.choice([rng.randrange(0x80, 0x3000), rng.randrange(0x10000, 0x20000)]))
                            for _ in range(30)).encode("utf-8", errors="ignore")
        got = G.pretokenize(text)
        assert b"".join(got) == text and all(got)
        assert got == R.split(text), text


# ---------------------------------------------------------------- encode / decode

def test_round_trips(trained):
    ref, tok = trained
    info = tok.info
    assert (info.kind, info.vocab_size, info.n_merges, info.n_specials) == (2, 700, len(ref.merges), 1)
    assert info.eos_id == 256 + len(ref.merges) == tok.special_id(EOT)
    assert tok.special_id(b"<eos>") is None
    for hx in CASES["round_trips"]:
        s = H(hx)
        ids = tok.encode(s)
        assert tok.decode(ids) == s
        assert ids.min(initial=0) >= 0 and ids.max(initial=0) < 700
        assert tok.decode(tok.encode(s, with_specials=False)) == s
        assert ids.tolist() == ref.encode(s)
    rng = random.Random(11)
    for trial in range(300):
        s = random_bytes(rng, rng.randrange(300))
        if trial % 3 == 0:
            s += EOT + random_bytes(rng, 5)
        ids = tok.encode(s)
        assert tok.decode(ids) == s and ids.tolist() == ref.encode(s)


def test_special_tokens(trained):
    ref, tok = trained
    eos = tok.info.eos_id
    assert tok.encode(EOT).tolist() == [eos]
    assert tok.encode(EOT + EOT).tolist() == [eos, eos]
    adjacent = tok.encode(b"x" + EOT + b"y").tolist()
    assert len(adjacent) == 3 and adjacent[1] == eos
    ordinary = tok.encode(EOT, with_specials=False).tolist()
    assert len(ordinary) > 1 and max(ordinary) < eos
    more = G.Tokenizer.from_merges(ref.merges, [EOT, b"<|sep|>"])
    assert more.info.fingerprint != tok.info.fingerprint
    sep = more.special_id(b"<|sep|>")
    assert sep == 700 and more.encode(b"a<|sep|>b" + EOT).tolist() == [ord("a"), sep, ord("b"), eos]
    o = CASES["overlapping_specials"]
    overlap = G.Tokenizer.from_merges([], [H(s) for s in o["specials"]])
    for c in o["cases"]:
        assert overlap.encode(H(c["text"])).tolist() == [256 + int(i[1:]) for i in c["ids"]]


def test_encode_matches_merge_order(trained):
    ref, tok = trained
    rng = random.Random(5)
    for trial in range(200):
        s = corpus(rng.randrange(1 << 30), 30)
        # long pieces take the heap path
        if trial % 4 == 0:
            s += b" " + b"a" * (40 + rng.randrange(40))
        if trial % 4 == 1:
            s += b" " * (30 + rng.randrange(30)) + b"x"
        if trial % 4 == 2:
            s += random_bytes(rng, 64)
        if trial % 4 == 3:
            s += b" supercalifragilisticexpialidocious_is_a_long_word"
        assert tok.encode(s, with_specials=False).tolist() == ref.encode_ordinary(s)
    assert tok.encode(b" little", with_specials=False).tolist() == ref.encode_ordinary(b" little")


def test_frozen_fingerprint():
    for f in CASES["frozen_fingerprints"]:
        tok = G.Tokenizer.from_merges(f["merges"], [H(s) for s in f["specials"]])
        assert f"{tok.info.fingerprint:016x}" == f["fingerprint"]


def test_fingerprint_matches_oracle(trained):
    ref, tok = trained
    assert tok.info.fingerprint == ref.fingerprint()


# ---------------------------------------------------------------- files

def test_save_load_byte_for_byte(trained, tmp_path):
    ref, tok = trained
    path = tmp_path / "tok.tok"
    tok.save(path)
    assert path.read_bytes() == ref.file_image()  # the layout grad.cpp writes
    loaded = G.Tokenizer.load(path)
    assert loaded.info.fingerprint == tok.info.fingerprint
    sample = corpus(8, 500)
    assert np.array_equal(loaded.encode(sample), tok.encode(sample))
    again = tmp_path / "again.tok"
    loaded.save(again)
    assert again.read_bytes() == path.read_bytes()


def test_corrupt_files(tmp_path):
    ref = R.train(corpus(4, 800), 300)
    good = ref.file_image()
    bad = tmp_path / "bad.tok"

    def why(data):
        bad.write_bytes(data)
        with pytest.raises(RuntimeError) as e:
            G.Tokenizer.load(bad)
        msg = str(e.value)
        assert msg.startswith(f"Tokenizer file {bad}: "), msg
        return msg[len(f"Tokenizer file {bad}: "):]

    def with_u32(offset, v):
        return good[:offset] + int(v).to_bytes(4, "little") + good[offset + 4:]

    bad.write_bytes(good)
    G.Tokenizer.load(bad)
    for n in range(4, len(good)):
        assert why(good[:n]).startswith("truncated reading "), n
    assert why(good + b"x") == "unexpected bytes after the fingerprint"
    assert why(with_u32(4, 3)) == "unsupported version 3"
    assert why(with_u32(8, 99)) == "unknown pre-tokenizer id 99"
    assert why(with_u32(12, 301)).startswith("implausible header: vocab 301, ")
    assert why(with_u32(16, 0xFFFFFFF0)).startswith("implausible header")
    assert why(with_u32(20, 5000)).startswith("implausible header")
    assert why(with_u32(24, 256)) == "special token 0 has id 256; special ids follow the merges"
    assert why(with_u32(28, 0)) == "special token 0 has an implausible length (0 bytes)"
    assert why(with_u32(28, 0x7FFFFFFF)).startswith("special token 0 has an implausible length")
    merges_at = 32 + len(EOT)
    assert why(with_u32(merges_at, 256)) == \
        f"merge 0 joins tokens 256 and {ref.merges[0][1]}, which it does not follow"
    changed = why(with_u32(merges_at + 8, 98))
    assert changed in ("fingerprint does not match the contents (corrupt file)",) or "repeats an earlier merge" in changed
    flipped = good[:-1] + bytes([good[-1] ^ 1])
    assert why(flipped) == "fingerprint does not match the contents (corrupt file)"
    # a file that does not start with the magic is taken for a v1 cache (tokenizer.cpp:107-124)
    bad.write_bytes(b"GTOX" + good[4:])
    with pytest.raises(RuntimeError, match="Tokenizer cache has an implausible vocab size"):
        G.Tokenizer.load(bad)
    with pytest.raises(RuntimeError, match="Failed to open tokenizer file: "):
        G.Tokenizer.load(tmp_path / "missing.tok")


def test_constructor_and_decode_errors(trained):
    ref, tok = trained
    with pytest.raises(ValueError, match="merge 0 joins tokens 300 and 1, which it does not follow"):
        G.Tokenizer.from_merges([(300, 1)], [])
    with pytest.raises(ValueError, match="merge 1 repeats an earlier merge"):
        G.Tokenizer.from_merges([(97, 98), (97, 98)], [])
    with pytest.raises(ValueError, match="special token 'x' is listed twice"):
        G.Tokenizer.from_merges([], [b"x", b"x"])
    with pytest.raises(ValueError, match="special token 0 has 0 bytes; allowed 1 to 1024"):
        G.Tokenizer.from_merges([], [b""])
    with pytest.raises(IndexError, match="token id 700 is outside the vocabulary of 700"):
        tok.decode([700])
    with pytest.raises(IndexError, match="token id -1 is outside the vocabulary of 700"):
        tok.decode([-1])
