"""The v1 whitespace BPE tokenizer of the library (cache reader, encoder, decoder,
fingerprint) against the CPU restatement in oracle/tokenizer_ref.py.  grad.cpp's golden ids
for v1 need a cache file that is a release download; what its golden cases fix without that
file (the decoded strings, tests/unit/test_tokenizer.cpp:604-640) is checked here on a
synthetic vocabulary.  Needs no GPU."""
import os
import random
import struct
import sys

import numpy as np
import pytest

import gradhip as G

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import tokenizer_ref as R  # noqa: E402

TEXT = (b"Once upon a time, there was a little girl named Lily.\nShe loved to play outside. "
        b"Hello world foo bar baz Tom said, \"I'm happy!\" 123 ... <|endoftext|> The end. "
        b"the cat sat on the mat and the cat ran to the hat " * 3)


@pytest.fixture(scope="module")
def v1(tmp_path_factory):
    ref = R.train_v1(TEXT + b"caf\xc3\xa9 \x98\x80", 220)
    path = tmp_path_factory.mktemp("v1") / "tok.cache"
    rng = random.Random(3)
    order = list(range(ref.vocab_size))
    rng.shuffle(order)   # grad.cpp writes its hash map's order: any order must load
    path.write_bytes(ref.cache_image(order))
    return ref, G.Tokenizer.load(path), path


def test_oracle_words_and_decoded_strings_of_the_reference_cases():
    """What tests/unit/test_tokenizer.cpp:604-625 fixes for every v1 vocabulary."""
    assert R.v1_words(b"Hello   world\tfoo_bar  baz\r\n") == [b"Hello", b"_world", b"_foo_bar", b"_baz"]
    assert R.v1_words(b"") == [] and R.v1_words(b" \n\t ") == []
    ref = R.train_v1(TEXT + b"caf\xc3\xa9 \x98\x80", 220)
    cases = {
        b"Once upon a time": b"Once upon a time",
        b"Once upon a time, there was a little girl named Lily.\nShe loved to play outside.":
            b"Once upon a time, there was a little girl named Lily. She loved to play outside.",
        b"Hello   world\tfoo_bar  baz\r\n": b"Hello world foo bar baz",
        b"<|endoftext|> The end.": b"<|endoftext|> The end.",
        b"": b"",
        # the emoji's bytes f0 9f are not in the vocabulary, 98 80 are
        b"Tom said, \"I'm happy!\" 123 ... caf\xc3\xa9 \xf0\x9f\x98\x80":
            b"Tom said, \"I'm happy!\" 123 ... caf\xc3\xa9 <unk><unk>\x98\x80",
    }
    for text, decoded in cases.items():
        assert ref.decode(ref.encode(text)) == decoded, text


def test_info_and_specials(v1):
    ref, tok, path = v1
    info = tok.info
    assert (info.kind, info.vocab_size, info.n_merges, info.n_specials) == (1, ref.vocab_size, len(ref.merges), 3)
    assert info.eos_id == 1 and tok.special_id(b"<unk>") == 2 and tok.special_id(b"<pad>") == 0
    assert tok.special_id(b"<|endoftext|>") is None and tok.special_id(b"the") is None
    assert info.fingerprint == ref.fingerprint()


def test_encode_decode_match_the_oracle(v1):
    ref, tok, path = v1
    rng = random.Random(9)
    words = TEXT.split()
    for trial in range(300):
        parts = []
        for _ in range(rng.randrange(0, 30)):
            w = rng.choice(words)
            if rng.random() < 0.2:
                w = bytes(rng.randrange(1, 256) for _ in range(rng.randrange(1, 8)))  # unknown bytes too
            parts.append(w + rng.choice([b" ", b"  ", b"\n", b"\t", b"\r\n", b" \x0b\x0c "]))
        text = b"".join(parts)
        ids = tok.encode(text)
        assert ids.tolist() == ref.encode(text), text
        assert tok.decode(ids) == ref.decode(ids)
    assert tok.encode(b"").tolist() == [] and tok.decode([]) == b""
    assert tok.decode([10 ** 6, -5]) == b""   # unknown ids are skipped (bpe_tokenizer.cpp:276-279)
    assert tok.encode(b"x", with_specials=False).tolist() == ref.encode(b"x")


def test_merge_list_order_is_literal():
    """The same string can be built by two merges; the list is walked once, in order, so a later
    merge never fires before an earlier one (bpe_tokenizer.cpp:222-247)."""
    vocab = list(R.V1_SPECIALS) + [(bytes([c]), 3 + i) for i, c in enumerate(b"_abcd")]
    for t in (b"bc", b"abc", b"ab", b"abcd"):
        vocab.append((t, len(vocab)))
    # (a,bc) comes after (ab,c) could have acted; ("abc","d") precedes the merge that builds "abc" from ab + c
    merges = [(b"b", b"c"), (b"abc", b"d"), (b"a", b"bc"), (b"a", b"b"), (b"ab", b"c")]
    ref = R.BpeV1Ref(vocab, merges)
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        p = os.path.join(d, "t.cache")
        open(p, "wb").write(ref.cache_image())
        tok = G.Tokenizer.load(p)
        for text in (b"abcd", b"abc abcd ab", b"aabcdd bcd"):
            assert tok.encode(text).tolist() == ref.encode(text), text
        # "abcd": b+c, then a+bc -> [abc, d]; the merge (abc, d) has already been passed
        assert [ref.id_to_token[i] for i in ref.encode(b"abcd")] == [b"abc", b"d"]


def test_save_reloads_with_the_same_identity(v1, tmp_path):
    ref, tok, path = v1
    again = tmp_path / "again.cache"
    tok.save(again)
    assert G.Tokenizer.load(again).info.fingerprint == ref.fingerprint()
    assert again.read_bytes() == R.BpeV1Ref(sorted(ref.vocab.items(), key=lambda kv: kv[1]), ref.merges).cache_image()


def test_corrupt_caches(v1, tmp_path):
    ref, tok, path = v1
    good = path.read_bytes()
    bad = tmp_path / "bad.cache"

    def why(data):
        bad.write_bytes(data)
        with pytest.raises(RuntimeError) as e:
            G.Tokenizer.load(bad)
        return str(e.value)

    assert why(b"") == f"Tokenizer cache truncated reading vocab size: {bad}"
    assert why(good[:11]) == f"Tokenizer cache truncated reading token length: {bad}"
    assert why(struct.pack("<Q", 1 << 30)) == f"Tokenizer cache has an implausible vocab size ({1 << 30}): {bad}"
    assert why(struct.pack("<QQ", 1, 1 << 20)) == \
        f"Tokenizer cache has an implausible token length ({1 << 20} bytes): {bad}"
    assert why(struct.pack("<QQ", 1, 5) + b"ab") == f"Tokenizer cache truncated reading a token: {bad}"
    assert why(struct.pack("<QQ", 1, 1) + b"a" + struct.pack("<i", -1)) == \
        f"Tokenizer cache has a negative token id: {bad}"
    assert why(struct.pack("<QQ", 1, 1) + b"a" + struct.pack("<i", 3)) == \
        f"Tokenizer cache truncated reading merge count: {bad}"
    for n in range(0, len(good), 7):
        assert "truncated" in why(good[:n]), n
