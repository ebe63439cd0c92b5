"""The tokenizer (J/Tokenizer.java): the library's host code against the oracle's Python restatement, both against
merges worked by hand on a tiny vocabulary and, when the reference's tokenizer.bin is at hand, against token ids of
the Llama-2 vocabulary that are public knowledge."""
import os
import struct

import numpy as np
import pytest

import llama2j_amd as l2j
from llama2j_amd.binding import L2JError
from oracle import tokenizer_ref as ref

REAL = "/root/reference/tokenizer/tokenizer.bin"
need_real = pytest.mark.skipif(not os.path.exists(REAL), reason="the reference's tokenizer.bin is not on this machine")


def write_tokenizer(path, entries):
    with open(path, "wb") as f:
        f.write(struct.pack("<i", max(len(s.encode("utf-8")) for _, s in entries)))
        for score, s in entries:
            b = s.encode("utf-8")
            f.write(struct.pack("<fi", score, len(b)) + b)


# ids 0..2 as in llama2.c's export, then the 256 byte tokens, then pieces
TINY = ([(0.0, "<unk>"), (0.0, "\n<s>\n"), (0.0, "\n</s>\n")] + [(0.0, "<0x%02X>" % b) for b in range(256)] +
        [(-1.0, " "), (-2.0, "a"), (-3.0, "b"), (-4.0, "c"), (-5.0, "é"), (-0.5, "ab"), (-0.25, " a"), (-0.75, "bc"),
         (-0.1, " ab"), (-6.0, "abc"), (-7.0, "b"), (-8.0, "😀"), (-9.0, "<0x>"), (-9.0, "<0x141>"), (-9.0, "<0xFFFFFFFFF>"),
         (-9.0, " <0x41>"), (-9.0, "<0x7fffffe9>")])
ID = {s: i for i, (_, s) in reversed(list(enumerate(TINY)))}     # first occurrence wins, as the reference's scan


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("tok") / "tokenizer.bin")
    write_tokenizer(path, TINY)
    return l2j.Tokenizer(path, len(TINY)), ref.Tokenizer(path, len(TINY))


def test_merges_worked_by_hand(tiny):
    for t in tiny:
        # " " a b c: candidates " a" (-0.25), "ab" (-0.5), "bc" (-0.75): " a" wins; then " a"+"b" = " ab" (-0.1) beats "bc";
        # then " ab"+"c": no such piece -> done
        assert list(t.bpe_encode("abc")) == [ID[" ab"], ID["c"]]
        # " " b c: " b" is no piece, "bc" merges
        assert list(t.bpe_encode("bc")) == [ID[" "], ID["bc"]]
        assert list(t.bpe_encode("")) == [ID[" "]]
        # the duplicate "b" (a later id) is never produced by the per-character scan
        assert ID["b"] in list(t.bpe_encode("b"))
        # a character missing from the vocabulary falls back to its bytes + 3 (ASCII only: 'z' = 0x7a)
        assert list(t.bpe_encode("z")) == [ID[" "], 0x7A + 3]
        # "é" is a piece of one char: found; two-unit pieces are not found char by char: each surrogate becomes '?'
        assert list(t.bpe_encode("é")) == [ID[" "], ID["é"]]
        assert list(t.bpe_encode("😀")) == [ID[" "], 0x3F + 3, 0x3F + 3]


def test_byte_fallback_above_0x7f_fails_as_in_the_reference(tiny):
    lib_tok, ref_tok = tiny
    with pytest.raises(L2JError):
        lib_tok.bpe_encode("ü")           # bytes C3 BC are negative Java bytes: ids -58, -65
    with pytest.raises(ref.JavaIndexError):
        ref_tok.bpe_encode("ü")


def test_decode_rules(tiny):
    for t in tiny:
        assert t.bpe_decode(5, ID[" ab"]) == " ab"
        assert t.bpe_decode(1, ID[" ab"]) == "ab"                       # the blank after BOS goes
        assert t.bpe_decode(1, ID["ab"]) == "ab"
        assert t.bpe_decode(7, 3 + 0x41) == "A"                         # raw byte token
        assert t.bpe_decode(7, 3 + 0x0A) == "\n"
        assert t.bpe_decode(7, 3 + 0x09) is None                        # control codes are dropped
        assert t.bpe_decode(7, 3 + 0x7F) is None and t.bpe_decode(7, 3 + 0x9F) is None
        assert t.bpe_decode(7, 3 + 0xE9) == "é"                         # a Latin-1 character, not a byte
        assert t.bpe_decode(7, ID["<0x>"]) is None                      # parseInt("") throws
        assert t.bpe_decode(7, ID["<0x141>"]) == "A"                    # value & 0xFF
        assert t.bpe_decode(7, ID["<0xFFFFFFFFF>"]) is None             # does not fit an int
        assert t.bpe_decode(7, ID["<0x7fffffe9>"]) == "é"
        assert t.bpe_decode(7, ID[" <0x41>"]) == " <0x41>"              # the pattern must match the whole string ...
        assert t.bpe_decode(1, ID[" <0x41>"]) == "A"                    # ... which it does once the blank is stripped
        assert t.bpe_decode(7, ID["😀"]) == "😀"


def test_library_equals_restatement_on_random_prompts(tiny):
    lib_tok, ref_tok = tiny
    rng = np.random.default_rng(0)
    alphabet = list("abc é") + ["z", "😀", "\n"]
    for _ in range(300):
        s = "".join(rng.choice(alphabet, size=int(rng.integers(0, 12))))
        assert list(lib_tok.bpe_encode(s)) == ref_tok.bpe_encode(s), repr(s)
    for nxt in range(len(TINY)):
        for tok in (1, 2):
            assert lib_tok.bpe_decode(tok, nxt) == ref_tok.bpe_decode(tok, nxt), (tok, nxt)


def test_open_errors(tmp_path):
    with pytest.raises(L2JError):
        l2j.Tokenizer(str(tmp_path / "missing.bin"), 10)
    p = str(tmp_path / "short.bin")
    write_tokenizer(p, TINY[:20])
    with pytest.raises(L2JError):
        l2j.Tokenizer(p, 30)


@need_real
def test_llama2_vocabulary_known_ids():
    lib_tok, ref_tok = l2j.Tokenizer(REAL, 32000), ref.Tokenizer(REAL, 32000)
    for t in (lib_tok, ref_tok):
        assert list(t.bpe_encode("Hello world")) == [15043, 3186]
        assert list(t.bpe_encode("Once upon a time")) == [9038, 2501, 263, 931]
        assert t.bpe_decode(1, 15043) == "Hello" and t.bpe_decode(15043, 3186) == " world"
        assert t.bpe_decode(2, 13) == "\n"                       # <0x0A>
    for s in ("The quick brown fox jumps over the lazy dog.", "  two  blanks", "1 + 1 = 2\n", "naïve café", "汉字 テスト"):
        try:
            want = ref_tok.bpe_encode(s)
        except ref.JavaIndexError:
            with pytest.raises(L2JError):
                lib_tok.bpe_encode(s)
            continue
        got = list(lib_tok.bpe_encode(s))
        assert got == want, s
        text = "".join(x for x in (lib_tok.bpe_decode(a, b) for a, b in zip([1] + got[:-1], got)) if x is not None)
        assert text == s, (s, text)
    for nxt in range(0, 32000, 7):
        assert lib_tok.bpe_decode(3, nxt) == ref_tok.bpe_decode(3, nxt)
