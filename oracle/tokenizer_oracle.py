"""Pure-Python restatement of the reference tokenizer (llama2.c's BPE).

TEST INFRASTRUCTURE ONLY: imported by tests/ as the checker of tensorlib_amd/host/tokenizer.cpp; the product
never imports it.  Small inputs only (the merge loop is quadratic, as in the reference).

Follows model/llama2_7b/src/Tokenizer.cpp:
  read_tokenizer_file  <- Tokenizer::Tokenizer  :7-60
  encode               <- Tokenizer::encode     :62-154
  decode_piece         <- Tokenizer::decode     :156-169
Pinned in tests/test_tokenizer.py by hand-worked merge sequences on a small vocabulary, by the round trip
decode(encode(text)) == text, and by the byte-fallback identity (a character outside the vocabulary becomes
its UTF-8 bytes + 3).
"""
from __future__ import annotations

import re
import struct


def read_tokenizer_file(path: str, vocab_size: int):
    pieces, scores = [], []
    with open(path, "rb") as f:
        (max_len,) = struct.unpack("<i", f.read(4))
        for _ in range(vocab_size):
            score, n = struct.unpack("<fi", f.read(8))
            scores.append(score)
            pieces.append(f.read(n))
    return pieces, scores, max_len


def encode(pieces, scores, text: bytes, bos: bool, eos: bool):
    index = {}
    for i, p in enumerate(pieces):
        index.setdefault(p, i)
    tokens = []
    if bos:
        tokens.append(1)
    if text and b" " in index:
        tokens.append(index[b" "])          # dummy prefix (Tokenizer.cpp:86-89)
    i = 0
    while i < len(text):                    # one UTF-8 character at a time (Tokenizer.cpp:96-124)
        j = i + 1
        while j < len(text) and (text[j] & 0xC0) == 0x80 and j - i < 4:
            j += 1
        ch = text[i:j]
        if ch in index:
            tokens.append(index[ch])
        else:
            tokens.extend(b + 3 for b in ch)
        i = j
    while True:                             # best-scoring adjacent pair, first wins ties (Tokenizer.cpp:128-149)
        best = None
        for k in range(len(tokens) - 1):
            pid = index.get(pieces[tokens[k]] + pieces[tokens[k + 1]])
            if pid is not None and scores[pid] > (best[0] if best else -1e10):
                best = (scores[pid], pid, k)
        if best is None:
            break
        tokens[best[2]:best[2] + 2] = [best[1]]
    if eos:
        tokens.append(2)
    return tokens


def decode_piece(pieces, prev_token: int, token: int) -> bytes:
    piece = pieces[token]
    if prev_token == 1 and piece[:1] == b" ":
        piece = piece[1:]
    m = re.fullmatch(rb"<0x([0-9A-Fa-f]{2})>", piece)
    if m:
        piece = bytes([int(m.group(1), 16)])
    return piece
