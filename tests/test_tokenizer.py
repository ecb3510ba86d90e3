"""The llama2.c-format tokenizer (tensorlib_amd/host/tokenizer.cpp) against its Python restatement and against
hand-worked cases.  Host-side only: runs without a GPU.  The reference ships no tokenizer.bin and no tokenizer
test, so vocabularies are synthetic (written in the reference's file format by write_tokenizer_file)."""
import os

import numpy as np
import pytest

from oracle import tokenizer_oracle as tor
from tensorlib_amd._lib import TensorLibError
from tensorlib_amd.tokenizer import Tokenizer, write_tokenizer_file


def base_vocab():
    """ids 0..2 specials, 3..258 byte tokens, as in the Llama2 sentencepiece vocabulary."""
    pieces = [b"<unk>", b"\n<s>\n", b"\n</s>\n"] + [f"<0x{b:02X}>".encode() for b in range(256)]
    scores = [0.0] * len(pieces)
    return pieces, scores


def small_vocab():
    pieces, scores = base_vocab()
    extra = [(b" ", -1.0), (b"a", -2.0), (b"b", -3.0), (b"c", -4.0), (b"ab", -0.5), (b" a", -0.7), (b" ab", -0.2),
             (b"abc", -0.9), (b"bc", -0.1), ("é".encode(), -5.0), (b" c", -6.0)]
    for p, s in extra:
        pieces.append(p)
        scores.append(s)
    return pieces, scores


@pytest.fixture()
def small(tmp_path):
    pieces, scores = small_vocab()
    path = str(tmp_path / "tok.bin")
    write_tokenizer_file(path, pieces, scores)
    return Tokenizer(path, len(pieces)), pieces, scores


def ids(pieces, *names):
    return [pieces.index(n) for n in names]


def test_hand_worked_merges(small):
    tok, pieces, scores = small
    # "ab": [" ", "a", "b"] -> candidates " a" (-0.7), "ab" (-0.5): "ab" wins -> [" ", "ab"] -> " ab" (-0.2)
    assert tok.encode("ab", bos=True, eos=False) == [1] + ids(pieces, b" ab")
    # "abc": [" ","a","b","c"]: " a" -0.7, "ab" -0.5, "bc" -0.1 -> "bc" first -> [" ","a","bc"]; then " a" -0.7
    # (a+bc = "abc" -0.9 loses) -> [" a","bc"]; " abc" is not in the vocabulary -> done
    assert tok.encode("abc", bos=False, eos=True) == ids(pieces, b" a", b"bc") + [2]
    # "ca": [" ","c","a"]: " c" -6.0 is the only candidate -> [" c","a"]
    assert tok.encode("ca", bos=False, eos=False) == ids(pieces, b" c", b"a")
    # empty text: no dummy prefix, only the requested specials (Tokenizer.cpp:86-89)
    assert tok.encode("", bos=True, eos=True) == [1, 2]
    assert tok.encode("", bos=False, eos=False) == []


def test_utf8_grouping_and_byte_fallback(small):
    tok, pieces, scores = small
    e = "é".encode()
    assert tok.encode("é", bos=False) == ids(pieces, b" ", e)                # two-byte character found whole
    z = "ž".encode()                                                          # not in the vocabulary: bytes + 3
    assert tok.encode("ž", bos=False) == ids(pieces, b" ") + [z[0] + 3, z[1] + 3]
    four = "𝄞".encode()                                                      # four-byte character
    assert tok.encode("𝄞", bos=False) == ids(pieces, b" ") + [b + 3 for b in four]
    # a stray continuation byte is a character of its own; five continuation bytes split after four
    assert tok.encode(b"\x80", bos=False) == ids(pieces, b" ") + [0x80 + 3]
    assert tok.encode(b"a\x80\x80\x80\x80", bos=False)[-4:] == [0x80 + 3] * 4


def test_decode_rules(small):
    tok, pieces, scores = small
    sp_ab = pieces.index(b" ab")
    assert tok.decode_piece(1, sp_ab) == b"ab"          # leading space dropped after BOS
    assert tok.decode_piece(5, sp_ab) == b" ab"
    assert tok.decode_piece(1, sp_ab) == b"ab"          # and the stored piece was not altered by the first call
    assert tok.decode_piece(-1, 3 + 0x0A) == b"\n"      # byte token
    assert tok.decode_piece(-1, 3 + 0xE2) == b"\xe2"
    with pytest.raises(TensorLibError, match="outside"):
        tok.decode_piece(-1, len(pieces))
    with pytest.raises(TensorLibError, match="outside"):
        tok.decode_piece(-1, -1)


def random_vocab(rng, n_merges):
    """A vocabulary grown the way BPE training grows one: new pieces are concatenations of existing ones."""
    pieces, scores = base_vocab()
    alphabet = [b" ", b"e", b"t", b"a", b"o", b"n", "é".encode(), "中".encode(), b"\n"]
    for a in alphabet:
        pieces.append(a)
        scores.append(float(-100 - len(pieces)))
    grown = list(alphabet)
    for m in range(n_merges):
        p = grown[rng.integers(len(grown))] + grown[rng.integers(len(grown))]
        if p in pieces or len(p) > 12:
            continue
        pieces.append(p)
        scores.append(float(-m) + float(rng.integers(0, 3)))   # repeated scores exercise the first-wins tie rule
        grown.append(p)
    return pieces, scores


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_matches_the_restatement_on_random_vocabularies(tmp_path, seed):
    rng = np.random.default_rng(seed)
    pieces, scores = random_vocab(rng, 300)
    path = str(tmp_path / "tok.bin")
    write_tokenizer_file(path, pieces, scores)
    got_pieces, got_scores, max_len = tor.read_tokenizer_file(path, len(pieces))
    assert got_pieces == pieces and max_len == max(len(p) for p in pieces)
    assert np.array_equal(np.float32(got_scores), np.float32(scores))
    tok = Tokenizer(path, len(pieces))
    chars = [" ", "e", "t", "a", "o", "n", "é", "中", "\n", "x", "ž", "𝄞"]
    for case in range(60):
        text = "".join(chars[i] for i in rng.integers(0, len(chars), rng.integers(0, 40)))
        raw = text.encode()
        for bos, eos in ((True, False), (False, True)):
            want = tor.encode(pieces, scores, raw, bos, eos)
            got = tok.encode(text, bos=bos, eos=eos)
            assert got == want, (seed, case, text)
        toks = tok.encode(text, bos=True, eos=True)
        # round trip: the dummy prefix space is dropped again by the decode-after-BOS rule
        assert tok.decode(toks) == raw, (seed, case, text)
        prev = -1
        for t in toks:
            assert tok.decode_piece(prev, t) == tor.decode_piece(pieces, prev, t)
            prev = t


def test_load_errors(tmp_path):
    pieces, scores = small_vocab()
    path = str(tmp_path / "tok.bin")
    write_tokenizer_file(path, pieces, scores)
    with pytest.raises(TensorLibError, match="cannot open"):
        Tokenizer(str(tmp_path / "missing.bin"), 10)
    with pytest.raises(TensorLibError, match="truncated"):
        Tokenizer(path, len(pieces) + 1)                 # file holds fewer tokens than asked for
    data = open(path, "rb").read()
    short = str(tmp_path / "short.bin")
    open(short, "wb").write(data[: len(data) - 2])
    with pytest.raises(TensorLibError, match="truncated"):
        Tokenizer(short, len(pieces))
    with pytest.raises(TensorLibError, match="vocab_size"):
        Tokenizer(path, 0)
    assert Tokenizer(path, 100).vocab_size == 100        # a prefix of the file is a valid smaller vocabulary


def test_vocabulary_without_byte_tokens_is_reported(tmp_path):
    path = str(tmp_path / "tiny.bin")
    write_tokenizer_file(path, [b"<unk>", b"<s>", b"</s>", b" ", b"a"], [0, 0, 0, -1, -2])
    tok = Tokenizer(path, 5)
    assert tok.encode("a", bos=False) == [3, 4]
    with pytest.raises(TensorLibError, match="byte tokens"):
        tok.encode("b", bos=False)
