"""CPU restatement of the reference's byte-level BPE tokenizer (src/tokenizer.rs). TEST INFRASTRUCTURE:
only tests may import this file; the product is homura_amd/csrc/host/tokenizer.cpp.

Pinned by the reference's own known answers (src/tokenizer.rs:170-218: "Hello world" -> [15496, 995],
"Hello, world!" -> [15496, 11, 995, 0], [15496] -> "Hello", round trips) on its own vocabulary files.
The pre-tokeniser pattern is handed to the `regex` module as the reference hands it to fancy-regex.
"""
import json

import regex

# src/tokenizer.rs:71-74
PATTERN = regex.compile(
    r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+")


def bytes_to_unicode():
    """src/tokenizer.rs:19-41"""
    bs = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAC + 1)) + list(range(0xAE, 0xFF + 1))
    cs = bs[:]
    n = 0
    for b in range(256):
        if b not in bs:
            bs.append(b)
            cs.append(256 + n)
            n += 1
    return {b: chr(c) for b, c in zip(bs, cs)}


class Tokenizer:
    def __init__(self, vocab_path, merges_path):
        """src/tokenizer.rs:44-82"""
        with open(vocab_path, encoding="utf-8") as f:
            self.encoder = json.load(f)
        self.decoder = {v: k for k, v in self.encoder.items()}
        self.ranks = {}
        with open(merges_path, encoding="utf-8") as f:
            lines = [l for l in f.read().splitlines() if l and not l.startswith("#")]
        for rank, line in enumerate(lines):
            a, _, b = line.partition(" ")
            self.ranks[(a, b)] = rank
        self.byte_encoder = bytes_to_unicode()
        self.byte_decoder = {c: b for b, c in self.byte_encoder.items()}

    def bpe(self, token):
        """src/tokenizer.rs:85-116: the first occurrence of the lowest-ranked pair, one merge per round"""
        word = list(token)
        while len(word) > 1:
            best, best_rank = None, None
            for i in range(len(word) - 1):
                r = self.ranks.get((word[i], word[i + 1]))
                if r is not None and (best_rank is None or r < best_rank):
                    best, best_rank = i, r
            if best is None:
                break
            word[best:best + 2] = [word[best] + word[best + 1]]
        return word

    def pre_tokenize(self, text):
        return [m.group(0) for m in PATTERN.finditer(text)]

    def encode(self, text):
        """src/tokenizer.rs:119-144"""
        ids = []
        for piece in self.pre_tokenize(text):
            mapped = "".join(self.byte_encoder[b] for b in piece.encode("utf-8"))
            ids += [self.encoder[p] for p in self.bpe(mapped) if p in self.encoder]
        return ids

    def decode(self, ids):
        """src/tokenizer.rs:147-159"""
        text = "".join(self.decoder[i] for i in ids if i in self.decoder)
        raw = bytes(self.byte_decoder[c] for c in text if c in self.byte_decoder)
        return raw.decode("utf-8", errors="replace")
