"""The byte-level BPE tokenizer (reference src/tokenizer.rs) on the reference's own vocabulary files:
its known answers on the oracle restatement and on the library, and the library against the oracle on
text that exercises every alternative of the pre-tokeniser pattern. CPU only."""
import random
import sys
import unicodedata
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "oracle"))
FIX = ROOT / "tests" / "golden" / "gpt2_bpe"


@pytest.fixture(scope="module")
def oracle_tok():
    import bpe_tokenizer
    return bpe_tokenizer.Tokenizer(FIX / "vocab.json", FIX / "merges.txt")


@pytest.fixture(scope="module")
def tok():
    from homura_amd.tokenizer import Tokenizer
    with Tokenizer(FIX / "vocab.json", FIX / "merges.txt") as t:
        yield t


# src/tokenizer.rs:170-218
KNOWN = [("Hello world", [15496, 995]), ("Hello, world!", [15496, 11, 995, 0]), ("", [])]
ROUND_TRIPS = ["The quick brown fox jumps over the lazy dog.", "12345", "café résumé naïve"]


@pytest.mark.parametrize("which", ["oracle", "library"])
def test_reference_known_answers(which, oracle_tok, tok):
    t = oracle_tok if which == "oracle" else tok
    for text, ids in KNOWN:
        assert t.encode(text) == ids
    assert t.decode([15496]) == "Hello"
    for text in ROUND_TRIPS:
        ids = t.encode(text)
        assert ids and t.decode(ids) == text


def test_vocabulary_and_byte_alphabet(oracle_tok, tok):
    assert tok.vocab_size == len(oracle_tok.encoder) == 50257
    # every byte value has its own single-symbol token in this vocabulary: all 256 survive a round trip
    every = bytes(range(256)).decode("latin-1")
    assert tok.decode(tok.encode(every)) == every == oracle_tok.decode(oracle_tok.encode(every))


TEXTS = [
    "I'm sure they'll say it's what we'd've done, isn't it? HE'S, SHE'LL, 'Twas 'round",
    "  leading spaces,   runs   of   spaces and trailing   ",
    "line one\nline two\r\n\r\n  indented\n\n\n   \t\n x",
    "tabs\tand no-break em spaces　ideographic",
    "numbers 1 12 123 1234 12345678 3.14159 1,000,000 ٣٤٥ ⅓ ²",
    "symbols !!! ... --- <<<>>> $%^&*() [brackets] {braces} #hash @at ~tilde `tick`\n\nafter",
    "mixed:abc123def 456ghi _under_score camelCaseWord snake_case_word",
    "unicode: naïve façade Ünïcödé Ελληνικά Русский язык 中文字符 日本語テキスト 한국어 עברית العربية हिन्दी",
    "emoji 😀😃 👍🏽 flags 🇺🇳 and ‼ ⁉ ™ © ®",
    "a", " ", "\n", "'", "''s", "x's'S", "ſ's 'ſ", "end with space ", "end with newline\n", "\r\n", " \n ", "\t\t",
    "don't stop'til you get enough'",
]


def _assigned(cp):
    return unicodedata.category(chr(cp)) not in ("Cn", "Cs", "Co") and not (0x1C <= cp <= 0x1F)


def _random_texts(n, seed):
    rng = random.Random(seed)
    pools = [list(range(0x20, 0x7F)), [0x0A, 0x0D, 0x09, 0x20, 0x20, 0x20, 0xA0, 0x2003, 0x3000],
             [cp for cp in range(0xA1, 0x250) if _assigned(cp)], [cp for cp in range(0x370, 0x530) if _assigned(cp)],
             [cp for cp in range(0x4E00, 0x4E80)], [cp for cp in range(0x1F600, 0x1F640)], list(b"'stTrReEvVmMlLdD'")]
    out = []
    for _ in range(n):
        k = rng.randint(1, 60)
        out.append("".join(chr(rng.choice(rng.choice(pools))) for _ in range(k)))
    return out


def test_pre_tokeniser_matches_the_pattern(oracle_tok):
    from homura_amd.tokenizer import pre_tokenize
    for text in TEXTS + _random_texts(400, 1):
        assert pre_tokenize(text) == oracle_tok.pre_tokenize(text), repr(text)


def test_encode_and_decode_match_the_oracle(oracle_tok, tok):
    for text in TEXTS + _random_texts(300, 2):
        want = oracle_tok.encode(text)
        got = tok.encode(text)
        assert got == want, repr(text)
        assert tok.decode(got) == oracle_tok.decode(want)


def test_decode_of_partial_utf8_and_unknown_ids(oracle_tok, tok):
    ids = tok.encode("é😀")          # bytes C3 A9 F0 9F 98 80
    assert ids == oracle_tok.encode("é😀")
    for cut in range(len(ids) + 1):  # prefixes end inside a multi-byte character: U+FFFD, like from_utf8_lossy
        assert tok.decode(ids[:cut]) == oracle_tok.decode(ids[:cut])
        assert tok.decode(ids[cut:]) == oracle_tok.decode(ids[cut:])
    assert tok.decode([15496, 10 ** 6, 995]) == "Hello world"   # ids outside the vocabulary are dropped
    assert tok.decode([]) == ""


def test_open_errors():
    from homura_amd.tokenizer import Tokenizer
    with pytest.raises(ValueError, match="cannot open"):
        Tokenizer(FIX / "missing.json", FIX / "merges.txt")
    with pytest.raises(ValueError, match="JSON"):
        Tokenizer(FIX / "merges.txt", FIX / "merges.txt")
