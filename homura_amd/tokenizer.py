"""The reference's byte-level BPE tokenizer (src/tokenizer.rs) through the library's host code.
No GPU needed."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _ffi


def pre_tokenize(text: str) -> list[str]:
    """The pieces the reference's pattern (src/tokenizer.rs:71-74) cuts `text` into."""
    lib = _ffi.load()
    raw = text.encode("utf-8")
    n = lib.hm_tokenizer_pieces(raw, len(raw), None, 0)
    if n < 0:
        raise ValueError(f"hm_tokenizer_pieces: {n}")
    ends = np.zeros(max(n, 1), np.uintp)
    lib.hm_tokenizer_pieces(raw, len(raw), ends.ctypes.data, n)
    out, at = [], 0
    for e in ends[:n]:
        out.append(raw[at:int(e)].decode("utf-8", errors="replace"))
        at = int(e)
    return out


class Tokenizer:
    """reference Tokenizer (src/tokenizer.rs:6-158)."""

    def __init__(self, vocab_json, merges_txt):
        self.lib = _ffi.load()
        err = C.create_string_buffer(512)
        self.h = self.lib.hm_tokenizer_open(str(vocab_json).encode(), str(merges_txt).encode(), err, 512)
        if not self.h:
            raise ValueError(err.value.decode())

    def close(self):
        if self.h:
            self.lib.hm_tokenizer_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def vocab_size(self) -> int:
        return self.lib.hm_tokenizer_vocab_size(self.h)

    def encode(self, text: str) -> list[int]:
        raw = text.encode("utf-8")
        ids = np.zeros(max(len(raw), 1), np.uint32)        # a piece of BPE never yields more ids than bytes
        n = self.lib.hm_tokenizer_encode(self.h, raw, len(raw), ids.ctypes.data, ids.size)
        if n < 0 or n > ids.size:
            raise ValueError(f"hm_tokenizer_encode: {n}")
        return ids[:n].tolist()

    def decode(self, ids) -> str:
        ids = np.ascontiguousarray(ids, np.uint32).reshape(-1)
        n = self.lib.hm_tokenizer_decode(self.h, ids.ctypes.data if ids.size else None, ids.size, None, 0)
        if n < 0:
            raise ValueError(f"hm_tokenizer_decode: {n}")
        buf = C.create_string_buffer(max(n, 1))
        self.lib.hm_tokenizer_decode(self.h, ids.ctypes.data if ids.size else None, ids.size, buf, n)
        return buf.raw[:n].decode("utf-8")
