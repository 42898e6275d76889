"""CPU restatement of grad.cpp's byte-level BPE tokenizer.  TEST INFRASTRUCTURE ONLY:
nothing in the library imports this file; tests compare the library against it.

What it follows and what pins it:

* split(): GPT-2's pre-tokenizer pattern (grad.cpp include/grad/tokenizer/pretokenize.h:5-9,
  src/tokenizer/pretokenize.cpp:104-167) run by the third-party `regex` module
  (the same oracle grad.cpp's own tests name, tests/unit/test_tokenizer.cpp:179-183),
  not a hand-written matcher, so it is independent of the library's matcher.
  Invalid UTF-8 bytes become lone surrogates (surrogateescape), one scalar of
  class "other" each, as pretokenize.cpp:53-90 treats them.  Pinned by the golden
  splits of tests/unit/test_tokenizer.cpp:184-241 (tests/golden/tokenizer_cases.json).
  The `regex` module carries its own Unicode database (17.0 with regex 2026.7.19);
  grad.cpp's tables are Unicode 16.0.0, so the letters and digits that 17.0 added
  (AGE_17, from the standard's DerivedAge data) are taken out of the letter and number classes
  here; the endpoints of those ranges are pinned as class "other" by samples of
  grad.cpp's own table in tests/golden/tokenizer_cases.json.
* encode_ordinary(): merges applied in rank order, every occurrence left to right
  (the definition grad.cpp's tests check the fast encoder against,
  tests/unit/test_tokenizer.cpp:150-171).
* encode(): special tokens found left to right, earliest first, longest on a tie
  (src/tokenizer/byte_bpe.cpp:60-86, :567-585); pinned by the overlapping-specials
  cases of tests/unit/test_tokenizer.cpp:398-406.
* fingerprint(): FNV-1a 64 over length-prefixed little-endian fields
  (src/tokenizer/byte_io.h:78-101, src/tokenizer/byte_bpe.cpp:333-347); pinned by the
  published FNV-1a vectors and by the value grad.cpp's test freezes for
  ByteBpe({{97, 98}}, {"<|endoftext|>"}) (tests/unit/test_tokenizer.cpp:470).
* file_image() / parse_file(): the GTOK v2 layout (src/tokenizer/byte_bpe.cpp:655-744).
* train(): highest count first, ties to the smallest (left bytes, right bytes)
  (include/grad/tokenizer/byte_bpe.h:55-60); pinned by the tie-break cases of
  tests/unit/test_tokenizer.cpp:475-489.  Only used to make realistic merge lists
  for tests; the library does not train.
"""
import struct
from collections import Counter

import regex

# Letters and digits first assigned in Unicode 17.0 (unassigned, hence "other", in 16.0).
AGE_17 = [
    (0x088F, 0x088F), (0x0C5C, 0x0C5C), (0x0CDC, 0x0CDC), (0xA7CE, 0xA7CF), (0xA7D2, 0xA7D2), (0xA7D4, 0xA7D4),
    (0xA7F1, 0xA7F1), (0x10940, 0x10959), (0x10EC5, 0x10EC7), (0x11DB0, 0x11DDB), (0x11DE0, 0x11DE9),
    (0x16EA0, 0x16EB8), (0x16EBB, 0x16ED3), (0x16FF2, 0x16FF6), (0x187F8, 0x187FF), (0x18D09, 0x18D1E),
    (0x18D80, 0x18DF2), (0x1E6C0, 0x1E6DE), (0x1E6E0, 0x1E6E2), (0x1E6E4, 0x1E6E5), (0x1E6E7, 0x1E6ED),
    (0x1E6F0, 0x1E6F4), (0x1E6FE, 0x1E6FF), (0x2B73A, 0x2B73F), (0x2CEA2, 0x2CEAD), (0x323B0, 0x33479),
]
_NEW = "".join(f"\\U{lo:08X}-\\U{hi:08X}" for lo, hi in AGE_17)
LETTER_16 = rf"[\p{{L}}--[{_NEW}]]"
NUMBER_16 = rf"[\p{{N}}--[{_NEW}]]"
OTHER_16 = rf"[[^\s\p{{L}}\p{{N}}]||[{_NEW}]]"
# GPT-2's pattern with the classes of Unicode 16.0 ((?V1): set difference and union)
GPT2_PATTERN = regex.compile(
    rf"""(?V1)'s|'t|'re|'ve|'m|'ll|'d| ?{LETTER_16}+| ?{NUMBER_16}+| ?{OTHER_16}+|\s+(?!\S)|\s+""")
EOT = b"<|endoftext|>"


def split(text: bytes) -> list:
    s = text.decode("utf-8", errors="surrogateescape")
    return [p.encode("utf-8", errors="surrogateescape") for p in GPT2_PATTERN.findall(s)]


def fnv1a64(data: bytes, h: int = 0xcbf29ce484222325) -> int:
    for b in data:
        h = ((h ^ b) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
    return h


def _u32(v: int) -> bytes:
    return struct.pack("<I", v)


def _lp(s: bytes) -> bytes:
    return _u32(len(s)) + s


class ByteBpeRef:
    def __init__(self, merges, specials=(EOT,)):
        self.merges = [(int(a), int(b)) for a, b in merges]
        self.specials = [bytes(s) for s in specials]
        self.token_bytes = [bytes([b]) for b in range(256)]
        for r, (a, b) in enumerate(self.merges):
            assert 0 <= a < 256 + r and 0 <= b < 256 + r
            self.token_bytes.append(self.token_bytes[a] + self.token_bytes[b])
        self.token_bytes += self.specials

    @property
    def vocab_size(self):
        return len(self.token_bytes)

    def fingerprint(self) -> int:
        buf = _lp(b"grad.tokenizer.bytebpe") + _u32(2) + _u32(1) + _u32(len(self.specials))
        for s in self.specials:
            buf += _lp(s)
        buf += _u32(len(self.merges))
        for a, b in self.merges:
            buf += _u32(a) + _u32(b)
        return fnv1a64(buf)

    def encode_ordinary(self, text: bytes) -> list:
        out = []
        for piece in split(text):
            s = list(piece)
            for r, (a, b) in enumerate(self.merges):
                if len(s) < 2:
                    break
                merged, i = [], 0
                while i < len(s):
                    if i + 1 < len(s) and s[i] == a and s[i + 1] == b:
                        merged.append(256 + r)
                        i += 2
                    else:
                        merged.append(s[i])
                        i += 1
                s = merged
            out += s
        return out

    def encode(self, text: bytes) -> list:
        out, pos = [], 0
        first_special = 256 + len(self.merges)
        while True:
            best = None  # (position, -length, index)
            for i, sp in enumerate(self.specials):
                at = text.find(sp, pos)
                if at >= 0 and (best is None or (at, -len(sp)) < best[:2]):
                    best = (at, -len(sp), i)
            stop = len(text) if best is None else best[0]
            out += self.encode_ordinary(text[pos:stop])
            if best is None:
                return out
            out.append(first_special + best[2])
            pos = best[0] - best[1]

    def decode(self, ids) -> bytes:
        return b"".join(self.token_bytes[i] for i in ids)

    def file_image(self) -> bytes:
        buf = b"GTOK" + _u32(2) + _u32(1) + _u32(self.vocab_size) + _u32(len(self.merges)) + _u32(len(self.specials))
        for k, s in enumerate(self.specials):
            buf += _u32(256 + len(self.merges) + k) + _lp(s)
        for a, b in self.merges:
            buf += _u32(a) + _u32(b)
        return buf + struct.pack("<Q", self.fingerprint())


def parse_file(data: bytes) -> ByteBpeRef:
    assert data[:4] == b"GTOK"
    version, pre, vocab, n_merges, n_specials = struct.unpack_from("<5I", data, 4)
    assert (version, pre) == (2, 1) and vocab == 256 + n_merges + n_specials
    at, specials = 24, []
    for k in range(n_specials):
        sid, ln = struct.unpack_from("<2I", data, at)
        assert sid == 256 + n_merges + k
        specials.append(data[at + 8:at + 8 + ln])
        at += 8 + ln
    merges = [struct.unpack_from("<2I", data, at + 8 * r) for r in range(n_merges)]
    at += 8 * n_merges
    tok = ByteBpeRef(merges, specials)
    assert struct.unpack_from("<Q", data, at)[0] == tok.fingerprint() and at + 8 == len(data)
    return tok


def train(text: bytes, vocab_size: int, specials=(EOT,)) -> ByteBpeRef:
    """Learns vocab_size - 256 - len(specials) merges: each step joins the pair with the
    highest count over the multiset of pre-tokens, ties to the smallest (left bytes,
    right bytes); special tokens in the text are left out."""
    specials = [bytes(s) for s in specials]
    segments, pos = [], 0
    probe = ByteBpeRef([], specials)
    # cut the specials out the way encode() finds them
    while True:
        best = None
        for sp in specials:
            at = text.find(sp, pos)
            if at >= 0 and (best is None or (at, -len(sp)) < best):
                best = (at, -len(sp))
        stop = len(text) if best is None else best[0]
        segments.append(text[pos:stop])
        if best is None:
            break
        pos = best[0] - best[1]
    words = Counter()
    for seg in segments:
        for piece in split(seg):
            words[tuple(piece)] += 1
    token_bytes = list(probe.token_bytes[:256])
    merges = []
    while len(merges) < vocab_size - 256 - len(specials):
        pairs = Counter()
        for w, c in words.items():
            for i in range(len(w) - 1):
                pairs[(w[i], w[i + 1])] += c
        if not pairs:
            break
        (a, b), _ = min(pairs.items(), key=lambda kv: (-kv[1], token_bytes[kv[0][0]], token_bytes[kv[0][1]]))
        new = 256 + len(merges)
        merges.append((a, b))
        token_bytes.append(token_bytes[a] + token_bytes[b])
        nxt = Counter()
        for w, c in words.items():
            out, i = [], 0
            while i < len(w):
                if i + 1 < len(w) and w[i] == a and w[i + 1] == b:
                    out.append(new)
                    i += 2
                else:
                    out.append(w[i])
                    i += 1
            nxt[tuple(out)] += c
        words = nxt
    return ByteBpeRef(merges, specials)


# ---------------------------------------------------------------------------
# v1: the original whitespace BPE (grad.cpp src/tokenizer/bpe_tokenizer.cpp).
#
# What pins it: the reference's golden ids (tests/unit/test_tokenizer.cpp:604-640) need the
# TinyStories cache, a release download that is absent offline, so ids are PARITY UNPINNED.
# What those golden cases fix without the cache is used instead: the decoded strings
# (white-space runs collapse to one space, '_' reads back as a space, characters missing
# from the vocabulary come back as "<unk>", bytes 0x98 0x80 of an emoji survive when they
# are in the vocabulary) hold for any v1 vocabulary and are checked in tests/test_tokenizer_v1.py.

V1_SPECIALS = ((b"<pad>", 0), (b"<eos>", 1), (b"<unk>", 2))


def v1_words(text: bytes) -> list:
    """`stream >> word` (bpe_tokenizer.cpp:176-189): split at C-locale white space; every
    word but the first gets a leading '_'."""
    words = text.replace(b"\t", b" ").replace(b"\n", b" ").replace(b"\v", b" ").replace(b"\f", b" ") \
        .replace(b"\r", b" ").split(b" ")
    words = [w for w in words if w]
    return [w if i == 0 else b"_" + w for i, w in enumerate(words)]


class BpeV1Ref:
    def __init__(self, vocab, merges):
        """vocab: list of (token bytes, id); merges: list of (left bytes, right bytes)."""
        self.vocab = {}
        self.id_to_token = {}
        for tok, i in vocab:
            self.vocab[bytes(tok)] = int(i)
            self.id_to_token[int(i)] = bytes(tok)
        self.merges = [(bytes(a), bytes(b)) for a, b in merges]

    @property
    def vocab_size(self):
        return len(self.vocab)

    def encode(self, text: bytes) -> list:
        out = []
        for word in v1_words(text):
            parts = [bytes([c]) for c in word]
            for a, b in self.merges:   # the whole list, in order (bpe_tokenizer.cpp:222-247)
                if len(parts) <= 1:
                    break
                merged, i = [], 0
                while i < len(parts):
                    if i + 1 < len(parts) and parts[i] == a and parts[i + 1] == b:
                        merged.append(a + b)
                        i += 2
                    else:
                        merged.append(parts[i])
                        i += 1
                parts = merged
            out += [self.vocab.get(p, 2) for p in parts]
        return out

    def decode(self, ids) -> bytes:
        return b"".join(self.id_to_token.get(int(i), b"") for i in ids).replace(b"_", b" ")

    def fingerprint(self) -> int:
        """v1_fingerprint (src/tokenizer/tokenizer.cpp:39-60)."""
        buf = _lp(b"grad.tokenizer.bpe_v1") + _u32(len(self.id_to_token))
        for i in sorted(self.id_to_token):
            buf += _u32(i) + _lp(self.id_to_token[i])
        buf += _u32(len(self.merges))
        for a, b in self.merges:
            buf += _lp(a) + _lp(b)
        return fnv1a64(buf)

    def cache_image(self, order=None) -> bytes:
        """BPETokenizer::save (bpe_tokenizer.cpp:307-335) as a 64-bit little-endian host writes
        it; the vocabulary goes out in `order` (grad.cpp: its hash map's order)."""
        entries = list(self.vocab.items())
        if order is not None:
            entries = [entries[i] for i in order]
        buf = struct.pack("<Q", len(entries))
        for tok, i in entries:
            buf += struct.pack("<Q", len(tok)) + tok + struct.pack("<i", i)
        buf += struct.pack("<Q", len(self.merges))
        for a, b in self.merges:
            buf += struct.pack("<Q", len(a)) + a + struct.pack("<Q", len(b)) + b
        return buf


def train_v1(text: bytes, vocab_size: int) -> BpeV1Ref:
    """BPETokenizer::train (bpe_tokenizer.cpp:23-172) with a fixed tie-break (grad.cpp takes the
    first maximum in its hash map's order, which depends on the C++ library): three specials,
    the characters of the text in byte order with '_', then the most frequent adjacent pair of
    the word list again and again.  Makes test material; ids are not the reference's."""
    vocab = list(V1_SPECIALS)
    chars = sorted({b"_"} | {bytes([c]) for c in text if c != 0x20})
    for c in chars:
        vocab.append((c, len(vocab)))
    words = Counter(v1_words(text))
    parts = {w: [bytes([c]) for c in w] for w in words}
    merges = []
    have = {t for t, _ in vocab}
    while len(have) < vocab_size:
        pairs = Counter()
        for w, p in parts.items():
            for i in range(len(p) - 1):
                pairs[(p[i], p[i + 1])] += words[w]
        if not pairs:
            break
        (a, b), _ = min(pairs.items(), key=lambda kv: (-kv[1], kv[0]))
        merges.append((a, b))
        vocab.append((a + b, len(vocab)))
        have.add(a + b)
        for w, p in parts.items():
            out, i = [], 0
            while i < len(p):
                if i + 1 < len(p) and p[i] == a and p[i + 1] == b:
                    out.append(a + b)
                    i += 2
                else:
                    out.append(p[i])
                    i += 1
            parts[w] = out
    return BpeV1Ref(vocab, merges)
