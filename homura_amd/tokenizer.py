"""The reference's byte-level BPE tokenizer (src/tokenizer.rs) and its tokenizer.json wrapper
(src/hf/tokenizer.rs) through the library's host code. No GPU needed."""
from __future__ import annotations

import ctypes as C
import unicodedata

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
    """reference Tokenizer (src/tokenizer.rs:6-158) over vocab.json + merges.txt; from_tokenizer_json gives
    the reference's HfTokenizer (src/hf/tokenizer.rs:4-47) for tokenizer.json files of the byte-level and the
    SentencePiece-style (Llama-2) BPE families."""

    def __init__(self, vocab_json=None, merges_txt=None, *, tokenizer_json=None):
        self.lib = _ffi.load()
        err = C.create_string_buffer(1024)
        if tokenizer_json is not None:
            self.h = self.lib.hm_tokenizer_open_json(str(tokenizer_json).encode(), err, 1024)
        else:
            self.h = self.lib.hm_tokenizer_open(str(vocab_json).encode(), str(merges_txt).encode(), err, 1024)
        if not self.h:
            raise ValueError(err.value.decode(errors="replace"))
        # the library leaves the NFC normaliser of a tokenizer.json to its caller
        self._nfc = bool(self.lib.hm_tokenizer_wants_nfc(self.h) > 0)

    @classmethod
    def from_tokenizer_json(cls, path) -> "Tokenizer":
        """HfTokenizer::from_file (src/hf/tokenizer.rs:10-14)."""
        return cls(tokenizer_json=path)

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

    def token_to_id(self, token: str):
        """Id of a vocabulary entry or added token, None when there is none."""
        i = self.lib.hm_tokenizer_token_to_id(self.h, token.encode("utf-8"))
        return None if i < 0 else int(i)

    def _encode(self, text: str, add_special_tokens: bool) -> list[int]:
        if self._nfc:
            text = unicodedata.normalize("NFC", text)
        raw = text.encode("utf-8")
        ids = np.zeros(len(raw) + 16, np.uint32)  # BPE never yields more ids than bytes; room for a template
        n = self.lib.hm_tokenizer_encode_ex(self.h, raw, len(raw), int(add_special_tokens), ids.ctypes.data, ids.size)
        if n > ids.size:
            ids = np.zeros(n, np.uint32)
            n = self.lib.hm_tokenizer_encode_ex(self.h, raw, len(raw), int(add_special_tokens), ids.ctypes.data, ids.size)
        if n < 0:
            raise ValueError(f"hm_tokenizer_encode_ex: {n}")
        return ids[:n].tolist()

    def encode(self, text: str) -> list[int]:
        """Tokenizer::encode (src/tokenizer.rs:119-144) / HfTokenizer::encode (src/hf/tokenizer.rs:17-23)."""
        return self._encode(text, False)

    def encode_with_special(self, text: str) -> list[int]:
        """HfTokenizer::encode_with_special (src/hf/tokenizer.rs:41-47)."""
        return self._encode(text, True)

    def _decode(self, ids, skip_special: bool) -> str:
        ids = np.ascontiguousarray(ids, np.uint32).reshape(-1)
        p = ids.ctypes.data if ids.size else None
        n = self.lib.hm_tokenizer_decode_ex(self.h, p, ids.size, int(skip_special), None, 0)
        if n < 0:
            raise ValueError(f"hm_tokenizer_decode_ex: {n}")
        buf = C.create_string_buffer(max(n, 1))
        self.lib.hm_tokenizer_decode_ex(self.h, p, ids.size, int(skip_special), buf, n)
        return buf.raw[:n].decode("utf-8")

    def decode(self, ids) -> str:
        """Tokenizer::decode (src/tokenizer.rs:147-159) / HfTokenizer::decode (src/hf/tokenizer.rs:25-30):
        added tokens marked special are left out."""
        return self._decode(ids, True)

    def decode_raw(self, ids) -> str:
        """HfTokenizer::decode_raw (src/hf/tokenizer.rs:32-38): special tokens stay in the text."""
        return self._decode(ids, False)
