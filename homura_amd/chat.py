"""Chat templates, stop-token lookup and streaming decode around the tokenizer: the host-side pieces of the
reference's chat mode (src/hf/chat.rs, src/generate.rs:480-516). The reference renders templates with
minijinja; this module uses jinja2, which must be importable to render (loading a template does not need it)."""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

from .tokenizer import Tokenizer


@dataclass
class ChatMessage:
    """reference ChatMessage (src/hf/chat.rs:11-15)."""
    role: str
    content: str


def _token_text(value):
    """Special tokens are stored as strings or as {"content": "..."} objects (src/hf/chat.rs:41-52)."""
    if isinstance(value, str):
        return value
    if isinstance(value, dict) and isinstance(value.get("content"), str):
        return value["content"]
    return None


class ChatTemplate:
    """reference ChatTemplate (src/hf/chat.rs:18-116): the Jinja chat_template of tokenizer_config.json."""

    TOKEN_KEYS = ("eos_token", "bos_token", "unk_token", "pad_token")

    def __init__(self, template_source: str, special_tokens: dict | None = None):
        self.template_source = template_source
        self.special_tokens = dict(special_tokens or {})

    @classmethod
    def load(cls, model_dir) -> "ChatTemplate":
        """ChatTemplate::load (src/hf/chat.rs:26-59)."""
        path = Path(model_dir) / "tokenizer_config.json"
        try:
            config = json.loads(path.read_text(encoding="utf-8"))
        except OSError as e:
            raise ValueError(f"failed to read tokenizer_config.json: {e}") from e
        source = config.get("chat_template")
        if not isinstance(source, str):
            raise ValueError("no chat_template field in tokenizer_config.json")
        tokens = {}
        for key in cls.TOKEN_KEYS:
            text = _token_text(config.get(key))
            if text is not None:
                tokens[key] = text
        return cls(source, tokens)

    def render(self, messages, add_generation_prompt: bool, enable_thinking: bool | None = None) -> str:
        """ChatTemplate::render (src/hf/chat.rs:81-115). enable_thinking None leaves the variable undefined
        in the template, True / False define it."""
        import jinja2
        from jinja2.sandbox import ImmutableSandboxedEnvironment

        def raise_exception(message):
            raise jinja2.exceptions.TemplateError(message)

        env = ImmutableSandboxedEnvironment()  # minijinja's defaults: no block trimming
        env.globals["raise_exception"] = raise_exception
        template = env.from_string(self.template_source)
        context = {
            "messages": [{"role": m.role, "content": m.content} if isinstance(m, ChatMessage) else dict(m)
                         for m in messages],
            "add_generation_prompt": bool(add_generation_prompt),
        }
        context.update(self.special_tokens)
        if enable_thinking is not None:
            context["enable_thinking"] = bool(enable_thinking)
        return template.render(**context)


def find_think_tokens(tokenizer: Tokenizer):
    """find_think_tokens (src/hf/chat.rs:119-128): the ids of <think> and </think> when each is one token."""
    open_ids = tokenizer.encode_with_special("<think>")
    close_ids = tokenizer.encode_with_special("</think>")
    if len(open_ids) == 1 and len(close_ids) == 1:
        return open_ids[0], close_ids[0]
    return None


def find_chat_stop_token(model_dir, tokenizer: Tokenizer):
    """find_chat_stop_token (src/hf/chat.rs:134-165): eos_token of tokenizer_config.json when it is a single
    token, else <|im_end|>, else None."""
    try:
        config = json.loads((Path(model_dir) / "tokenizer_config.json").read_text(encoding="utf-8"))
    except (OSError, ValueError):
        return None

    def resolve(token: str):
        ids = tokenizer.encode_with_special(token)
        return ids[0] if len(ids) == 1 else None

    eos = _token_text(config.get("eos_token"))
    if eos is not None:
        found = resolve(eos)
        if found is not None:
            return found
    return resolve("<|im_end|>")


class StreamDecoder:
    """decode_streaming_token (src/generate.rs:480-516): text of one generated token at a time. Tokens that
    end inside a UTF-8 sequence decode to U+FFFD on their own; they are held back until the run decodes
    cleanly."""

    def __init__(self, tokenizer: Tokenizer, raw: bool = False):
        self._decode = tokenizer.decode_raw if raw else tokenizer.decode
        self._held: list[int] = []

    def push(self, token: int, prev_token: int | None = None) -> str:
        if not self._held:
            if prev_token is not None:
                combined, prefix = self._decode([prev_token, token]), self._decode([prev_token])
                text = combined[len(prefix):] if combined.startswith(prefix) else combined
            else:
                text = self._decode([token])
            if "�" in text:
                self._held.append(token)
                return ""
            return text
        self._held.append(token)
        text = self._decode(self._held)
        if "�" in text:
            return ""
        self._held.clear()
        return text
