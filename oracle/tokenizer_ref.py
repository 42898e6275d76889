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
  grad.cpp's tables are Unicode 16.0.0: code points first assigned after 16.0
  are "parity unpinned".
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

GPT2_PATTERN = regex.compile(
    r"""'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+""")
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
