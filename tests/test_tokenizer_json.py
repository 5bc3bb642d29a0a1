"""tokenizer.json files (the reference's HfTokenizer, src/hf/tokenizer.rs, a wrapper around the `tokenizers`
crate, 0.21.4 in its Cargo.lock) and the chat helpers (src/hf/chat.rs). The checker for the tokenizer is the
`tokenizers` Python package, a binding of that same crate: each test writes a tokenizer.json with it (the
reference's GPT-2 vocabulary and merges under the Qwen2 or the Llama-3 pre-tokeniser, with added tokens), loads
the file into the library and compares ids and text. CPU only."""
import json
import random
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
FIX = ROOT / "tests" / "golden" / "gpt2_bpe"

tokenizers = pytest.importorskip("tokenizers")

QWEN2 = ("(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\\r\\n\\p{L}\\p{N}]?\\p{L}+|\\p{N}| ?[^\\s\\p{L}\\p{N}]+[\\r\\n]*"
         "|\\s*[\\r\\n]+|\\s+(?!\\S)|\\s+")
LLAMA3 = QWEN2.replace("|\\p{N}|", "|\\p{N}{1,3}|")


def _base():
    vocab = json.loads((FIX / "vocab.json").read_text(encoding="utf-8"))
    lines = (FIX / "merges.txt").read_text(encoding="utf-8").split("\n")
    merges = [tuple(l.split(" ")) for l in lines if l and not l.startswith("#")]
    return vocab, merges


def _build(tmp_path, family):
    from tokenizers import AddedToken, Regex, Tokenizer, decoders, normalizers, pre_tokenizers, processors
    from tokenizers.models import BPE
    vocab, merges = _base()
    if family == "qwen2":
        t = Tokenizer(BPE(vocab=vocab, merges=merges))
        t.normalizer = normalizers.NFC()
        pattern = QWEN2
    else:
        t = Tokenizer(BPE(vocab=vocab, merges=merges, ignore_merges=True))
        pattern = LLAMA3
    t.pre_tokenizer = pre_tokenizers.Sequence([
        pre_tokenizers.Split(Regex(pattern), behavior="isolated", invert=False),
        pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)])
    t.decoder = decoders.ByteLevel()
    if family == "qwen2":
        t.post_processor = processors.ByteLevel(trim_offsets=False)
        t.add_special_tokens([AddedToken("<|im_start|>", special=True, normalized=False),
                              AddedToken("<|im_end|>", special=True, normalized=False),
                              AddedToken("<|im_end|><|extra|>", special=True, normalized=False)])
        t.add_tokens([AddedToken("<think>", special=False, normalized=False),
                      AddedToken("</think>", special=False, normalized=False)])
    else:
        t.add_special_tokens([AddedToken("<|begin_of_text|>", special=True, normalized=False),
                              AddedToken("<|eot_id|>", special=True, normalized=False)])
        bos = t.token_to_id("<|begin_of_text|>")
        t.post_processor = processors.Sequence([
            processors.ByteLevel(trim_offsets=False),
            processors.TemplateProcessing(single="<|begin_of_text|> $A", pair="<|begin_of_text|> $A <|begin_of_text|> $B:1",
                                          special_tokens=[("<|begin_of_text|>", bos)])])
    path = tmp_path / f"{family}.json"
    t.save(str(path))
    return t, path


TEXTS = [
    "", "Hello world", "Hello, world!", "The year 2024 had 366 days; pi = 3.14159265.",
    "<|im_start|>system\nYou are helpful.<|im_end|>\n<|im_start|>user\nHi there 12345!<|im_end|>\n<|im_start|>assistant\n",
    "<think>\n\n</think>\n\nSure's  it\r\n  x", "a<think>b</think>c <|im_end|>", "<|im_start|><|im_end|><|im_start",
    "<|im_end|><|extra|> then <|im_end|><|extr", "<|begin_of_text|>x<|eot_id|>", "<|eot_id|<|eot_id|>",
    "café naïve 日本語 🙂 don'T I'LL we'Ve 3.14159  \t\n\n  end ", "    indented\n\tcode();\r\n\r\n}", "ſ's 'ſ",
    "١٢٣٤٥ ½ ²³ 1234567 x9y", "a b c　d", "é vs é (combining)", "tab\tsep\t\tfields   ",
    " leading and trailing ", "\n\n\n", "   ", "!!!???...\n\n##", "I'm you're he'll they'd it's don't",
]


def _random_texts(n, seed):
    rng = random.Random(seed)
    alphabet = ("abcdefghijklmnopqrstuvwxyzABCDEFGHIJKLMNOPQRSTUVWXYZ" "0123456789" "    \t\n\r" ".,;:!?'\"()-_/\\#@"
                "éüßøçñ" "日本語中文" "١٢٣½" "🙂🚀" "  ")
    specials = ["<|im_start|>", "<|im_end|>", "<think>", "</think>", "<|eot_id|>", "<|begin_of_text|>", "<|im_", "<thi"]
    out = []
    for _ in range(n):
        parts = []
        for _ in range(rng.randint(1, 12)):
            if rng.random() < 0.2:
                parts.append(rng.choice(specials))
            else:
                parts.append("".join(rng.choice(alphabet) for _ in range(rng.randint(1, 12))))
        out.append("".join(parts))
    return out


@pytest.mark.parametrize("family", ["qwen2", "llama3"])
def test_ids_and_text_match_the_tokenizers_crate(tmp_path, family):
    from homura_amd.tokenizer import Tokenizer
    theirs, path = _build(tmp_path, family)
    with Tokenizer.from_tokenizer_json(path) as mine:
        assert mine.vocab_size == theirs.get_vocab_size(with_added_tokens=True)
        for text in TEXTS + _random_texts(300, 7):
            want = theirs.encode(text, add_special_tokens=False).ids
            assert mine.encode(text) == want, repr(text)
            want_sp = theirs.encode(text, add_special_tokens=True).ids
            assert mine.encode_with_special(text) == want_sp, repr(text)
            assert mine.decode(want_sp) == theirs.decode(want_sp, skip_special_tokens=True), repr(text)
            assert mine.decode_raw(want_sp) == theirs.decode(want_sp, skip_special_tokens=False), repr(text)
        for token in ("<|im_end|>", "<|eot_id|>", "<think>", "Hello", "Ġworld", "no such token"):
            assert mine.token_to_id(token) == theirs.token_to_id(token)


def test_template_prefix_only_with_special_tokens(tmp_path):
    from homura_amd.tokenizer import Tokenizer
    theirs, path = _build(tmp_path, "llama3")
    bos = theirs.token_to_id("<|begin_of_text|>")
    with Tokenizer.from_tokenizer_json(path) as mine:
        assert mine.encode("Hello world") == [15496, 995]
        assert mine.encode_with_special("Hello world") == [bos, 15496, 995]


def test_merges_as_strings_and_as_pairs(tmp_path):
    from homura_amd.tokenizer import Tokenizer
    _, path = _build(tmp_path, "qwen2")
    doc = json.loads(path.read_text(encoding="utf-8"))
    merges = doc["model"]["merges"]
    as_pairs = [m.split(" ") if isinstance(m, str) else m for m in merges]
    as_strings = [" ".join(m) for m in as_pairs]
    results = []
    for name, form in (("pairs", as_pairs), ("strings", as_strings)):
        doc["model"]["merges"] = form
        p = tmp_path / f"{name}.json"
        p.write_text(json.dumps(doc), encoding="utf-8")
        with Tokenizer.from_tokenizer_json(p) as t:
            results.append(t.encode("The quick brown fox jumps over 13 lazy dogs."))
    assert results[0] == results[1] and len(results[0]) > 5


def test_files_outside_the_family_are_refused(tmp_path):
    from homura_amd.tokenizer import Tokenizer
    _, path = _build(tmp_path, "qwen2")
    good = json.loads(path.read_text(encoding="utf-8"))

    def refused(change, needle):
        doc = json.loads(json.dumps(good))
        change(doc)
        p = tmp_path / "bad.json"
        p.write_text(json.dumps(doc), encoding="utf-8")
        with pytest.raises(ValueError) as e:
            Tokenizer.from_tokenizer_json(p)
        assert needle in str(e.value), str(e.value)

    refused(lambda d: d.__setitem__("pre_tokenizer", {"type": "ByteLevel", "add_prefix_space": False,
                                                         "trim_offsets": True, "use_regex": True}), "GPT-2")
    refused(lambda d: d["pre_tokenizer"]["pretokenizers"][0]["pattern"].__setitem__("Regex", "\\w+|\\s+"), "Split pattern")
    refused(lambda d: d["added_tokens"][0].__setitem__("lstrip", True), "lstrip")
    refused(lambda d: d["model"].__setitem__("type", "WordPiece"), "BPE")
    refused(lambda d: d["model"].__setitem__("byte_fallback", True), "byte_fallback")
    refused(lambda d: d.__setitem__("normalizer", {"type": "Lowercase"}), "normalizer")
    refused(lambda d: d.__setitem__("decoder", {"type": "WordPiece"}), "decoder")
    with pytest.raises(ValueError):
        Tokenizer.from_tokenizer_json(tmp_path / "missing.json")


def test_nfc_is_applied_by_the_wrapper(tmp_path):
    from homura_amd.tokenizer import Tokenizer
    theirs, path = _build(tmp_path, "qwen2")
    with Tokenizer.from_tokenizer_json(path) as mine:
        decomposed, composed = "café", "café"
        assert mine.encode(decomposed) == mine.encode(composed) == theirs.encode(decomposed, add_special_tokens=False).ids


# ── chat helpers ──────────────────────────────────────────────────────────────

CHATML = ("{%- for message in messages %}"
          "{{- '<|im_start|>' + message.role + '\\n' + message.content + '<|im_end|>\\n' }}"
          "{%- endfor %}"
          "{%- if add_generation_prompt %}"
          "{{- '<|im_start|>assistant\\n' }}"
          "{%- endif %}")


def test_render_chatml_basic():
    """src/hf/chat.rs:171-202"""
    from homura_amd.chat import ChatMessage, ChatTemplate
    t = ChatTemplate(CHATML)
    out = t.render([ChatMessage("system", "You are helpful."), ChatMessage("user", "Hello")], True, None)
    assert "<|im_start|>system\nYou are helpful.<|im_end|>" in out
    assert "<|im_start|>user\nHello<|im_end|>" in out
    assert out.endswith("<|im_start|>assistant\n")


def test_render_without_generation_prompt():
    """src/hf/chat.rs:204-226"""
    from homura_amd.chat import ChatMessage, ChatTemplate
    out = ChatTemplate(CHATML).render([ChatMessage("user", "Hi")], False, None)
    assert "<|im_start|>assistant" not in out


def test_template_variables_and_python_string_methods(tmp_path):
    """enable_thinking is undefined, true or false (src/hf/chat.rs:70-80); special tokens are template
    variables whether stored as strings or as objects (:38-52); templates use Python string methods."""
    from homura_amd.chat import ChatMessage, ChatTemplate
    source = ("{{ bos_token }}{% for m in messages %}{% if m.content.startswith('/') %}[cmd]{% endif %}"
              "{{ m.role }}:{{ m.content.strip() }}{{ eos_token }}{% endfor %}"
              "{% if enable_thinking is defined and enable_thinking is false %}<think>\n\n</think>{% endif %}"
              "{% if enable_thinking is not defined %}<undef>{% endif %}")
    (tmp_path / "tokenizer_config.json").write_text(json.dumps({
        "chat_template": source, "bos_token": "<s>", "eos_token": {"content": "</s>", "special": True},
        "pad_token": None}), encoding="utf-8")
    t = ChatTemplate.load(tmp_path)
    assert t.special_tokens == {"bos_token": "<s>", "eos_token": "</s>"}
    msgs = [ChatMessage("user", "  /go  ".strip() + " "), ChatMessage("assistant", " ok ")]
    assert t.render(msgs, False, None) == "<s>[cmd]user:/go</s>assistant:ok</s><undef>"
    assert t.render(msgs, False, False) == "<s>[cmd]user:/go</s>assistant:ok</s><think>\n\n</think>"
    assert t.render(msgs, False, True) == "<s>[cmd]user:/go</s>assistant:ok</s>"
    (tmp_path / "tokenizer_config.json").write_text("{}", encoding="utf-8")
    with pytest.raises(ValueError, match="no chat_template"):
        ChatTemplate.load(tmp_path)


def test_stop_and_think_tokens_and_delta_prefill(tmp_path):
    """find_chat_stop_token, find_think_tokens (src/hf/chat.rs:119-165) and the property the incremental
    prefill of chat mode rests on (docs/chat.md:34-45): the ids of a rendered conversation start with the ids
    of the same conversation one turn earlier."""
    from homura_amd.chat import ChatMessage, ChatTemplate, find_chat_stop_token, find_think_tokens
    from homura_amd.tokenizer import Tokenizer
    theirs, path = _build(tmp_path, "qwen2")
    with Tokenizer.from_tokenizer_json(path) as tok:
        assert find_think_tokens(tok) == (theirs.token_to_id("<think>"), theirs.token_to_id("</think>"))
        cfg = tmp_path / "tokenizer_config.json"
        cfg.write_text(json.dumps({"eos_token": {"content": "<|im_end|>"}}), encoding="utf-8")
        assert find_chat_stop_token(tmp_path, tok) == theirs.token_to_id("<|im_end|>")
        cfg.write_text(json.dumps({"eos_token": "not a single token"}), encoding="utf-8")
        assert find_chat_stop_token(tmp_path, tok) == theirs.token_to_id("<|im_end|>")  # the ChatML fallback
        assert find_chat_stop_token(tmp_path / "nowhere", tok) is None

        t = ChatTemplate(CHATML)
        turn1 = [ChatMessage("system", "Be brief."), ChatMessage("user", "2+2?")]
        ids1 = tok.encode_with_special(t.render(turn1, True, None))
        turn2 = turn1 + [ChatMessage("assistant", "4"), ChatMessage("user", "And 3+3?")]
        ids2 = tok.encode_with_special(t.render(turn2, True, None))
        assert ids2[:len(ids1)] == ids1 and len(ids2) > len(ids1)
    with Tokenizer(FIX / "vocab.json", FIX / "merges.txt") as plain:
        assert find_think_tokens(plain) is None


def test_stream_decoder_holds_back_split_characters(tmp_path):
    """decode_streaming_token (src/generate.rs:480-516)"""
    from homura_amd.chat import StreamDecoder
    from homura_amd.tokenizer import Tokenizer
    _, path = _build(tmp_path, "qwen2")
    with Tokenizer.from_tokenizer_json(path) as tok:
        text = "Hi 🙂 日本 ok<|im_end|>"
        ids = tok.encode(text)
        assert any("�" in tok.decode([i]) for i in ids)  # some token ends inside a character
        for raw, want in ((False, "Hi 🙂 日本 ok"), (True, text)):
            sd, out, prev = StreamDecoder(tok, raw=raw), [], None
            for i in ids:
                piece = sd.push(i, prev)
                assert "�" not in piece
                out.append(piece)
                prev = i
            assert "".join(out) == want
