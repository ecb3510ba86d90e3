"""ctypes binding of the llama2.c-format tokenizer in libtensorlib_llama2.so
(include/tensorlib_tokenizer.h).  Host-side only: text <-> token ids for the Llama2 driver."""
from __future__ import annotations

import ctypes
import struct
from typing import Iterable, Sequence

from ._lib import TensorLibError
from .llama2 import llama2_lib

_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
_PROTOS = {
    "tlt_last_error": (ctypes.c_char_p, []),
    "tlt_load": (_i, [ctypes.c_char_p, _i, ctypes.POINTER(_vp)]),
    "tlt_destroy": (_i, [_vp]),
    "tlt_vocab_size": (_i, [_vp]),
    "tlt_encode": (_i, [_vp, ctypes.c_char_p, _sz, _i, _i, ctypes.POINTER(_i), _sz, ctypes.POINTER(_sz)]),
    "tlt_decode": (_i, [_vp, _i, _i, ctypes.c_char_p, _sz, ctypes.POINTER(_sz)]),
}
_ready = False


def _l() -> ctypes.CDLL:
    global _ready
    h = llama2_lib()
    if not _ready:
        for name, (res, args) in _PROTOS.items():
            fn = getattr(h, name)
            fn.restype, fn.argtypes = res, args
        _ready = True
    return h


def _ck(status: int, what: str) -> None:
    if status != 0:
        raise TensorLibError(f"{what} failed: {_l().tlt_last_error().decode(errors='replace')}")


def write_tokenizer_file(path: str, pieces: Sequence[bytes], scores: Sequence[float]) -> None:
    """Writes a llama2.c tokenizer.bin: int32 max_token_length, then per token float32 score, int32 length, bytes."""
    with open(path, "wb") as f:
        f.write(struct.pack("<i", max((len(p) for p in pieces), default=0)))
        for p, s in zip(pieces, scores):
            f.write(struct.pack("<fi", s, len(p)))
            f.write(p)


class Tokenizer:
    """Tokenizer(path, vocab_size) with the reference's encode / decode (model/llama2_7b/src/Tokenizer.cpp:7-169)."""

    BOS, EOS = 1, 2

    def __init__(self, path: str, vocab_size: int):
        self.l = _l()
        h = _vp()
        _ck(self.l.tlt_load(path.encode(), vocab_size, ctypes.byref(h)), "tlt_load")
        self.h = h
        self.vocab_size = self.l.tlt_vocab_size(h)

    def __del__(self):
        if getattr(self, "h", None):
            self.l.tlt_destroy(self.h)
            self.h = None

    def encode(self, text: str | bytes, bos: bool = True, eos: bool = False) -> list[int]:
        raw = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        cap = len(raw) + 3
        buf = (_i * cap)()
        n = _sz(0)
        _ck(self.l.tlt_encode(self.h, raw, len(raw), int(bos), int(eos), buf, cap, ctypes.byref(n)), "tlt_encode")
        return list(buf[: n.value])

    def decode_piece(self, prev_token: int, token: int) -> bytes:
        buf = ctypes.create_string_buffer(256)
        n = _sz(0)
        rc = self.l.tlt_decode(self.h, prev_token, token, buf, len(buf), ctypes.byref(n))
        if rc != 0 and n.value > len(buf):
            buf = ctypes.create_string_buffer(n.value)
            rc = self.l.tlt_decode(self.h, prev_token, token, buf, len(buf), ctypes.byref(n))
        _ck(rc, "tlt_decode")
        return buf.raw[: n.value]

    def decode(self, tokens: Iterable[int]) -> bytes:
        """Concatenation of the pieces as Llama2::generate prints them; BOS and EOS ids themselves print nothing."""
        out, prev = [], -1
        for t in tokens:
            if t not in (self.BOS, self.EOS):
                out.append(self.decode_piece(prev, t))
            prev = t
        return b"".join(out)
