"""tokenizer.json files (the reference's HfTokenizer, src/hf/tokenizer.rs, a wrapper around the `tokenizers`
crate, 0.21.4 in its Cargo.lock) and the chat helpers (src/hf/chat.rs). The checker for the tokenizer is the
`tokenizers` Python package, a binding of that same crate: each test writes a tokenizer.json with it (the
reference's GPT-2 vocabulary and merges under the Qwen2 or the Llama-3 pre-tokeniser, with added tokens), loads
the file into the library and compares ids and text. The Llama-2 family (SentencePiece-style BPE with byte
fallback: TinyLlama, Mistral) gets a vocabulary trained by the package on a few lines, since no file of that
family is at hand. CPU only."""
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


SPM_CORPUS = [
    "The quick brown fox jumps over the lazy dog.", "Hello world, hello there, hello again!",
    "A tokenizer turns text into numbers and numbers back into text.", "It's 2024: 3 + 4 = 7, and 12345 * 2 = 24690.",
    "def main():\n    print('hello')\n    return 0", "caf\u00e9 na\u00efve r\u00e9sum\u00e9 \u00fcber stra\u00dfe",
    "the the the and and of of to to in in is is that that it it", "    indented   text  with   runs  of   spaces",
    "<s>[INST] What is the capital of France? [/INST] Paris.</s>", "one two three four five six seven eight nine ten",
] * 3


def _build_llama2(tmp_path, drop_bytes=()):
    """A tokenizer.json laid out as Llama-2's: BPE with unk_token, fuse_unk and byte_fallback over a vocabulary of
    pieces with U+2581 for spaces, no pre-tokeniser. `drop_bytes`: byte tokens left out of the vocabulary, so that
    characters with those bytes come out as the unknown token."""
    from tokenizers import Tokenizer, normalizers, trainers
    from tokenizers.models import BPE
    seed = Tokenizer(BPE())
    seed.normalizer = normalizers.Sequence([normalizers.Prepend("\u2581"), normalizers.Replace(" ", "\u2581")])
    seed.train_from_iterator(SPM_CORPUS, trainers.BpeTrainer(vocab_size=420, show_progress=False, special_tokens=[]))
    trained = json.loads(seed.to_str())["model"]
    pieces = sorted(trained["vocab"], key=trained["vocab"].get)
    # two characters of the corpus go to bytes instead; pieces that spell a special token would take its place
    pieces = [p for p in pieces if p not in ("\u00e9", "\u00df", "<unk>", "<s>", "</s>")]
    merges = [m if isinstance(m, list) else m.split(" ") for m in trained["merges"]]
    keep = set(pieces)
    merges = [m for m in merges if m[0] in keep and m[1] in keep and m[0] + m[1] in keep]
    names = ["<unk>", "<s>", "</s>"] + [f"<0x{b:02X}>" for b in range(256) if b not in drop_bytes] + pieces
    vocab = {name: i for i, name in enumerate(names)}
    special = [{"id": i, "content": c, "single_word": False, "lstrip": False, "rstrip": False, "normalized": False,
                "special": True} for i, c in enumerate(["<unk>", "<s>", "</s>"])]
    doc = {
        "version": "1.0", "truncation": None, "padding": None, "added_tokens": special,
        "normalizer": {"type": "Sequence", "normalizers": [
            {"type": "Prepend", "prepend": "\u2581"},
            {"type": "Replace", "pattern": {"String": " "}, "content": "\u2581"}]},
        "pre_tokenizer": None,
        "post_processor": {"type": "TemplateProcessing",
                           "single": [{"SpecialToken": {"id": "<s>", "type_id": 0}}, {"Sequence": {"id": "A", "type_id": 0}}],
                           "pair": [{"SpecialToken": {"id": "<s>", "type_id": 0}}, {"Sequence": {"id": "A", "type_id": 0}},
                                    {"SpecialToken": {"id": "<s>", "type_id": 1}}, {"Sequence": {"id": "B", "type_id": 1}}],
                           "special_tokens": {"<s>": {"id": "<s>", "ids": [1], "tokens": ["<s>"]}}},
        "decoder": {"type": "Sequence", "decoders": [
            {"type": "Replace", "pattern": {"String": "\u2581"}, "content": " "},
            {"type": "ByteFallback"}, {"type": "Fuse"}, {"type": "Strip", "content": " ", "start": 1, "stop": 0}]},
        "model": {"type": "BPE", "dropout": None, "unk_token": "<unk>", "continuing_subword_prefix": None,
                  "end_of_word_suffix": None, "fuse_unk": True, "byte_fallback": True, "ignore_merges": False,
                  "vocab": vocab, "merges": merges},
    }
    path = tmp_path / "llama2.json"
    path.write_text(json.dumps(doc), encoding="utf-8")
    return Tokenizer.from_file(str(path)), path


SPM_TEXTS = TEXTS + SPM_CORPUS[:10] + [
    "Hello</s>world", "<s>Hello</s> <s> again", " </s> ", "</s>", "<unk>known<unk>", "<0x0A> literal", "caf\u00e9\u00df\u00e9",
    "\U0001f642\U0001f680 and \u65e5\u672c", "\U0001f642a\U0001f642\u00e9\U0001f680\U0001f680b", "\u2581 already \u2581\u2581 there",
    "x" * 700 + " " + "the " * 300,
]


@pytest.mark.parametrize("drop_bytes", [(), tuple(range(0xF0, 0xF5)), (0x98, 0x99)], ids=["all_bytes", "no_f0_f4", "no_98_99"])
def test_llama2_family_matches_the_tokenizers_crate(tmp_path, drop_bytes):
    """Whole stretches between special tokens are one word; characters outside the vocabulary go in as byte tokens,
    or as one fused unknown token where a byte token is missing; decoding undoes both."""
    from homura_amd.tokenizer import Tokenizer
    theirs, path = _build_llama2(tmp_path, drop_bytes)
    rng = random.Random(11)
    strays = [[rng.randrange(theirs.get_vocab_size()) for _ in range(rng.randint(1, 10))] for _ in range(200)]
    strays += [[3 + 0xE6 - len([b for b in drop_bytes if b < 0xE6])], [1, 2, 0], []]
    with Tokenizer.from_tokenizer_json(path) as mine:
        assert mine.vocab_size == theirs.get_vocab_size(with_added_tokens=True)
        seen_unk = seen_byte = False
        for text in SPM_TEXTS + _random_texts(300, 13):
            want = theirs.encode(text, add_special_tokens=False).ids
            assert mine.encode(text) == want, repr(text)
            seen_unk |= 0 in want and "<unk>" not in text
            seen_byte |= any(3 <= i < 259 - len(drop_bytes) for i in want)
            want_sp = theirs.encode(text, add_special_tokens=True).ids
            assert mine.encode_with_special(text) == want_sp == [1] + want, repr(text)
            assert mine.decode(want_sp) == theirs.decode(want_sp, skip_special_tokens=True), repr(text)
            assert mine.decode_raw(want_sp) == theirs.decode(want_sp, skip_special_tokens=False), repr(text)
        assert seen_byte and seen_unk == bool(drop_bytes)
        for ids in strays:  # byte tokens that spell no UTF-8, in any company
            assert mine.decode(ids) == theirs.decode(ids, skip_special_tokens=True), ids
            assert mine.decode_raw(ids) == theirs.decode(ids, skip_special_tokens=False), ids
        for token in ("<s>", "</s>", "<0x0A>", "\u2581the", "no such token"):
            assert mine.token_to_id(token) == theirs.token_to_id(token)


def test_llama2_family_files_outside_it_are_refused(tmp_path):
    from homura_amd.tokenizer import Tokenizer
    _, path = _build_llama2(tmp_path)
    good = json.loads(path.read_text(encoding="utf-8"))

    def refused(change, needle):
        doc = json.loads(json.dumps(good))
        change(doc)
        p = tmp_path / "bad.json"
        p.write_text(json.dumps(doc), encoding="utf-8")
        with pytest.raises(ValueError) as e:
            Tokenizer.from_tokenizer_json(p)
        assert needle in str(e.value), str(e.value)

    refused(lambda d: d["model"].__setitem__("fuse_unk", False), "fuse_unk")
    refused(lambda d: d["model"].__setitem__("unk_token", None), "unk_token")
    refused(lambda d: d["model"].__setitem__("unk_token", "<nope>"), "unk_token")
    refused(lambda d: d["normalizer"]["normalizers"].pop(0), "normalizer")
    refused(lambda d: d["normalizer"]["normalizers"][0].__setitem__("prepend", "_"), "normalizer")
    refused(lambda d: d.__setitem__("normalizer", None), "normalizer")
    refused(lambda d: d.__setitem__("pre_tokenizer", {"type": "Whitespace"}), "pre-tokeniser")
    refused(lambda d: d["decoder"]["decoders"].pop(3), "decoder")
    refused(lambda d: d["decoder"]["decoders"][3].__setitem__("start", 0), "decoder")
    refused(lambda d: d["added_tokens"][1].__setitem__("normalized", True), "normalized")


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


def test_stream_decoder_on_the_llama2_family(tmp_path):
    """The decoder of this family drops one leading space from whatever it is handed, so a token's text is what it
    adds to the token before it (src/generate.rs:480-516); byte tokens of one character are held back together."""
    from homura_amd.chat import StreamDecoder
    from homura_amd.tokenizer import Tokenizer
    theirs, path = _build_llama2(tmp_path)
    with Tokenizer.from_tokenizer_json(path) as tok:
        for text in ("Hello world, hello there", "the caf\u00e9 \U0001f642 is  over there \u65e5\u672c ok", " two  spaces"):
            ids = tok.encode(text)
            assert ids == theirs.encode(text, add_special_tokens=False).ids
            sd, out, prev = StreamDecoder(tok), [], None
            for i in ids:
                piece = sd.push(i, prev)
                assert "\ufffd" not in piece
                out.append(piece)
                prev = i
            assert "".join(out) == text == tok.decode(ids)
