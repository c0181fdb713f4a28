"""Tokenizers: the model folder's tokenizer.json when it is there, else a byte tokenizer
so that folders of random weights can still be prompted with text.

The reference loads tokenizer.json and renders the chat template that tokenizer_config.json
carries (/root/reference/src/utils/mod.rs:1563-2086, src/utils/chat_template.rs:428-474); a
folder without one gets the default template of its architecture's family (the reference keeps
one per architecture too, /root/reference/src/utils/mod.rs:2297-2477).  Token ids remain the
engine's contract.
"""
from __future__ import annotations

import json
import os
from typing import List, Optional, Sequence


def render_chat_template(template: str, messages, bos_token: Optional[str] = None, eos_token: Optional[str] = None,
                         add_generation_prompt: bool = True, enable_thinking: bool = True) -> str:
    """Renders a chat template with the variables the reference hands to it
    (chat_template.rs:459-472: messages, add_generation_prompt, bos_token, eos_token,
    enable_thinking, tools) and its whitespace settings (lstrip_blocks, trim_blocks).  The
    template comes from a model folder, so it runs in jinja2's sandbox."""
    from jinja2.sandbox import ImmutableSandboxedEnvironment

    def raise_exception(message):
        raise ValueError(f"chat template: {message}")

    env = ImmutableSandboxedEnvironment(lstrip_blocks=True, trim_blocks=True)
    env.globals["raise_exception"] = raise_exception
    msgs = [{"role": m.role, "content": m.content} for m in messages]
    return env.from_string(template).render(
        messages=msgs, add_generation_prompt=add_generation_prompt, bos_token=bos_token, eos_token=eos_token,
        enable_thinking=enable_thinking, tools=[])


class IncrementalText:
    """Text of a growing token list, piece by piece: a piece is handed on only when it is final.
    A character that spans several tokens decodes to U+FFFD until its last token is there, so a
    text that ends in U+FFFD waits; a decoder may also join a token to the one before (a space it
    drops or adds), so each piece is what the tokens since the last piece add to the text of the
    few tokens before them, not the token's own text."""

    def __init__(self, tokenizer):
        self._tok = tokenizer
        self._prefix = 0          # tokens[_prefix:_read] are the context of the next piece
        self._read = 0            # tokens[:_read] are handed on

    def add(self, tokens: Sequence[int]) -> str:
        """`tokens`: all tokens so far.  Returns the text they add to what was handed on."""
        before = self._tok.decode(list(tokens[self._prefix:self._read]))
        now = self._tok.decode(list(tokens[self._prefix:]))
        if len(now) <= len(before) or now.endswith("\ufffd"):
            return ""
        self._prefix, self._read = self._read, len(tokens)
        return now[len(before):]

    def finish(self, tokens: Sequence[int]) -> str:
        """The text that `add` still holds back when the request ends: whatever the tokens since
        the last piece add, final or not (a request cut inside a character that spans several
        tokens ends in U+FFFD, as the text of all its tokens does)."""
        before = self._tok.decode(list(tokens[self._prefix:self._read]))
        now = self._tok.decode(list(tokens[self._prefix:]))
        self._prefix, self._read = self._read, len(tokens)
        return now[len(before):] if len(now) > len(before) else ""


class ByteTokenizer:
    """token = byte value modulo the vocabulary; decoding prints the ids."""

    def __init__(self, vocab_size: int):
        self.vocab_size = vocab_size

    def encode(self, text: str) -> List[int]:
        ids = [b % self.vocab_size for b in text.encode("utf-8")]
        return ids or [0]

    def decode(self, ids: Sequence[int]) -> str:
        return " ".join(f"<{i}>" for i in ids)

    def apply_chat_template(self, messages) -> str:
        return "\n".join(m.content for m in messages)

    def eos_token_ids(self) -> List[int]:
        return []


def _token_text(v) -> Optional[str]:
    if isinstance(v, dict):
        v = v.get("content")
    return v if isinstance(v, str) else None


class FileTokenizer:
    def __init__(self, model_dir: str, default_chat_template: Optional[str] = None):
        from tokenizers import Tokenizer
        self._tok = Tokenizer.from_file(os.path.join(model_dir, "tokenizer.json"))
        self._eos: List[int] = []
        self.bos_token = self.eos_token = None
        self.chat_template = default_chat_template
        cfg = os.path.join(model_dir, "tokenizer_config.json")
        if os.path.isfile(cfg):
            with open(cfg, "r", encoding="utf-8") as f:
                raw = json.load(f)
            self.bos_token, self.eos_token = _token_text(raw.get("bos_token")), _token_text(raw.get("eos_token"))
            if self.eos_token is not None:
                tid = self._tok.token_to_id(self.eos_token)
                if tid is not None:
                    self._eos.append(tid)
            if isinstance(raw.get("chat_template"), str):
                self.chat_template = raw["chat_template"]

    def encode(self, text: str) -> List[int]:
        return self._tok.encode(text, add_special_tokens=False).ids

    def decode(self, ids: Sequence[int]) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=True)

    def apply_chat_template(self, messages) -> str:
        if self.chat_template is None:
            raise ValueError("the model folder has no chat template and its architecture names no default")
        return render_chat_template(self.chat_template, messages, self.bos_token, self.eos_token)

    def eos_token_ids(self) -> List[int]:
        return list(self._eos)


def load_tokenizer(model_dir, vocab_size: int, default_chat_template: Optional[str] = None):
    """`model_dir` may be None (a model built in memory): the byte tokenizer."""
    if model_dir and os.path.isfile(os.path.join(model_dir, "tokenizer.json")):
        return FileTokenizer(model_dir, default_chat_template)
    return ByteTokenizer(vocab_size)
