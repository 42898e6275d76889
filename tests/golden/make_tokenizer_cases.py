"""Writes tokenizer_cases.json: the known answers grad.cpp's own tokenizer tests hold
(tests/unit/test_tokenizer.cpp), as data: golden pre-tokenizer splits (:184-241),
character classes (:256-281), UTF-8 decoding cases (:283-301), round-trip texts
(:326-350), special-token cases (:369-406), tie-break training cases (:475-489) and the
frozen fingerprint (:470).  Byte strings are stored as hex.

Run:  python tests/golden/make_tokenizer_cases.py
"""
import json
import os

SPLITS = [
    (b"Hello world", [b"Hello", b" world"]),
    (b"Hello  world", [b"Hello", b" ", b" world"]),
    (b"Hello   world", [b"Hello", b"  ", b" world"]),
    (b"a\nb", [b"a", b"\n", b"b"]),
    (b"a\n\nb", [b"a", b"\n", b"\n", b"b"]),
    (b"a \nb", [b"a", b" ", b"\n", b"b"]),
    (b"a\n\n", [b"a", b"\n\n"]),
    (b"  leading", [b" ", b" leading"]),
    (b"trailing  ", [b"trailing", b"  "]),
    (b"tab\tsep", [b"tab", b"\t", b"sep"]),
    (b"\t\tx", [b"\t", b"\t", b"x"]),
    (b"CRLF\r\nline", [b"CRLF", b"\r", b"\n", b"line"]),
    (b"don't", [b"don", b"'t"]),
    (b"I'm here", [b"I", b"'m", b" here"]),
    (b"they're", [b"they", b"'re"]),
    (b"we've", [b"we", b"'ve"]),
    (b"you'll", [b"you", b"'ll"]),
    (b"he'd", [b"he", b"'d"]),
    (b"it's", [b"it", b"'s"]),
    (b"IT'S", [b"IT", b"'", b"S"]),
    (b"'hello'", [b"'", b"hello", b"'"]),
    (b"!'s", [b"!'", b"s"]),
    (b"x 's", [b"x", b" '", b"s"]),
    (b"rock'n'roll", [b"rock", b"'", b"n", b"'", b"roll"]),
    (b"foo_bar baz", [b"foo", b"_", b"bar", b" baz"]),
    (b"__init__", [b"__", b"init", b"__"]),
    (b"a_b", [b"a", b"_", b"b"]),
    (b"123 4567 89", [b"123", b" 4567", b" 89"]),
    (b"abc123def", [b"abc", b"123", b"def"]),
    (b"3.14", [b"3", b".", b"14"]),
    (b" $5.00!", [b" $", b"5", b".", b"00", b"!"]),
    (b"...", [b"..."]),
    (b"?!", [b"?!"]),
    (b"\"Hi,\" she said.", [b"\"", b"Hi", b",\"", b" she", b" said", b"."]),
    (b"(a) [b] {c}", [b"(", b"a", b")", b" [", b"b", b"]", b" {", b"c", b"}"]),
    (b"e-mail", [b"e", b"-", b"mail"]),
    (b"--flag=value", [b"--", b"flag", b"=", b"value"]),
    (b"<|endoftext|>", [b"<|", b"endoftext", b"|>"]),
    (b"x\x0b\x0cy", [b"x", b"\x0b", b"\x0c", b"y"]),
    (b"\x1c\x1dz", [b"\x1c\x1d", b"z"]),
    (b" ", [b" "]),
    (b"", []),
    (b"caf\xc3\xa9", [b"caf\xc3\xa9"]),
    (b"e\xcc\x81", [b"e", b"\xcc\x81"]),
    (b"\xe6\x97\xa5\xe6\x9c\xac\xe8\xaa\x9e\xe3\x81\xa7\xe3\x81\x99",
     [b"\xe6\x97\xa5\xe6\x9c\xac\xe8\xaa\x9e\xe3\x81\xa7\xe3\x81\x99"]),
    (b"na\xc3\xafve r\xc3\xa9sum\xc3\xa9", [b"na\xc3\xafve", b" r\xc3\xa9sum\xc3\xa9"]),
    (b"\xc2\xa0nbsp", [b"\xc2\xa0", b"nbsp"]),
    (b"a\xe3\x80\x80b", [b"a", b"\xe3\x80\x80", b"b"]),
    (b"\xf0\x9f\x98\x80 smile", [b"\xf0\x9f\x98\x80", b" smile"]),
    (b"x\xc2\xb2 + \xc2\xbd", [b"x", b"\xc2\xb2", b" +", b" \xc2\xbd"]),
    (b"\xe2\x85\xa7 \xd9\xa3", [b"\xe2\x85\xa7", b" \xd9\xa3"]),
    (b"\xd9\x85\xd8\xb1\xd8\xad\xd8\xa8\xd8\xa7", [b"\xd9\x85\xd8\xb1\xd8\xad\xd8\xa8\xd8\xa7"]),
]

OTHER, LETTER, NUMBER, SPACE = 0, 1, 2, 3
CLASSES = [
    (ord("a"), LETTER), (ord("Z"), LETTER), (ord("7"), NUMBER), (ord("_"), OTHER), (ord("'"), OTHER),
    *[(ws, SPACE) for ws in (0x09, 0x0A, 0x0B, 0x0C, 0x0D, 0x20, 0x85, 0xA0, 0x1680, 0x2000, 0x200A, 0x2028,
                             0x2029, 0x202F, 0x205F, 0x3000)],
    (0x1C, OTHER), (0x200B, OTHER), (0xE9, LETTER), (0x0301, OTHER), (0x4E2D, LETTER), (0xB2, NUMBER),
    (0x2167, NUMBER), (0x0663, NUMBER), (0x1F600, OTHER), (0x10FFFF, OTHER),
]

# What grad.cpp's Unicode 16.0.0 class table (src/tokenizer/unicode_tables.h) says at the ends of
# the ranges that Unicode 17.0 filled with letters and digits: unassigned in 16.0, so "other";
# and at their assigned neighbours.
CLASSES += [(cp, OTHER) for cp in (
    0x088F, 0x0C5C, 0x0CDC, 0xA7CE, 0xA7CF, 0xA7D2, 0xA7D4, 0xA7F1, 0x10940, 0x10959, 0x10EC5, 0x10EC7, 0x11DB0,
    0x11DDB, 0x11DE0, 0x11DE9, 0x16EA0, 0x16EB8, 0x16EBB, 0x16ED3, 0x16FF2, 0x16FF6, 0x187F8, 0x187FF, 0x18D09,
    0x18D1E, 0x18D80, 0x18DF2, 0x1E6C0, 0x1E6DE, 0x1E6E0, 0x1E6E2, 0x1E6E4, 0x1E6E5, 0x1E6E7, 0x1E6ED, 0x1E6F0,
    0x1E6F4, 0x1E6FE, 0x1E6FF, 0x2B73A, 0x2B73F, 0x2CEA2, 0x2CEAD, 0x323B0, 0x33479)]
CLASSES += [(0x088E, LETTER), (0xA7CD, LETTER), (0xA7D3, LETTER), (0x187F7, LETTER), (0x18D08, LETTER),
            (0x2B739, LETTER), (0x2CEA1, LETTER), (0x323AF, LETTER), (0x3347A, OTHER), (0x10EC4, LETTER)]

# the first byte of each is one invalid scalar on its own
INVALID_UTF8 = [b"\xC0\xAF", b"\xE0\x80\xAF", b"\xED\xA0\x80", b"\xF4\x90\x80\x80", b"\xE6\x97", b"\x80", b"\xFF"]

ROUND_TRIPS = [
    b"", b"a", b"Hello world", b"   leading and trailing   ", b"tabs\tand\t\ttabs",
    b"lines\nand\n\n\nblank lines\n", b"CRLF\r\nline\r\n\r\n", b"literal_underscores __init__ _a_ ___",
    b"multi   spaces  \t \n mixed", b"caf\xc3\xa9 na\xc3\xafve \xe6\x97\xa5\xe6\x9c\xac\xe8\xaa\x9e",
    b"emoji \xf0\x9f\x98\x80\xf0\x9f\x91\x8d\xf0\x9f\x8f\xbd!",
    b"invalid \xff\xfe \xc0\xaf \xed\xa0\x80 \xe6\x97 \x80\x80", b"nul\0byte", b"<|endoftext|>",
    b"a<|endoftext|>b", b"<|endoftext|><|endoftext|><|endoftext|>", b"end.\n<|endoftext|>\nOnce upon",
    b"<|endoftext", b"<|endoftext|", b"<<|endoftext|>>", b" " * 1000, b"a" * 300 + b"\n" * 300,
]

# specials, text, expected ids as indices into the specials list (no merges: bytes are themselves)
OVERLAPPING_SPECIALS = {
    "specials": [b"<a>", b"<a><b>", b"b>"],
    "cases": [(b"<a><b>", ["s1"]), (b"<a>b>", ["s0", "s2"])],
}

# text, vocab size, specials, expected merges
TIE_BREAKS = [
    (b"ab\nac", 258, [], [(97, 98), (97, 99)]),
    (b"ab ab cd", 260, [], [(97, 98), (32, 256), (32, 99), (258, 100)]),
    (b"zb\n\xc3\xa9b", 259, [], [(122, 98), (0xA9, 98), (0xC3, 257)]),
]

FROZEN_FINGERPRINTS = [
    {"merges": [(97, 98)], "specials": [b"<|endoftext|>"], "fingerprint": "08b0b6b208dca2a9"},
]


def hx(b):
    return b.hex()


def main():
    data = {
        "splits": [{"text": hx(t), "pieces": [hx(p) for p in ps]} for t, ps in SPLITS],
        "classes": [{"codepoint": cp, "class": c} for cp, c in CLASSES],
        "invalid_utf8": [hx(b) for b in INVALID_UTF8],
        "round_trips": [hx(b) for b in ROUND_TRIPS],
        "overlapping_specials": {
            "specials": [hx(s) for s in OVERLAPPING_SPECIALS["specials"]],
            "cases": [{"text": hx(t), "ids": ids} for t, ids in OVERLAPPING_SPECIALS["cases"]],
        },
        "tie_breaks": [{"text": hx(t), "vocab": v, "specials": [hx(s) for s in sp], "merges": m}
                       for t, v, sp, m in TIE_BREAKS],
        "frozen_fingerprints": [{"merges": f["merges"], "specials": [hx(s) for s in f["specials"]],
                                 "fingerprint": f["fingerprint"]} for f in FROZEN_FINGERPRINTS],
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tokenizer_cases.json")
    with open(path, "w") as f:
        json.dump(data, f, indent=1)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
