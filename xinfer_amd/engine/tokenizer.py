"""Tokenizers: the model folder's tokenizer.json when it is there, else a byte tokenizer
so that folders of random weights can still be prompted with text.

The reference loads tokenizer.json and renders a chat template
(/root/reference/src/utils/mod.rs:1563-2086, src/utils/chat_template.rs); here the ChatML
form that Qwen3 uses is written out, and token ids remain the engine's contract.
"""
from __future__ import annotations

import json
import os
from typing import List, Sequence


def _chatml(messages) -> str:
    out = []
    for m in messages:
        out.append(f"<|im_start|>{m.role}\n{m.content}<|im_end|>\n")
    out.append("<|im_start|>assistant\n")
    return "".join(out)


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


class FileTokenizer:
    def __init__(self, model_dir: str):
        from tokenizers import Tokenizer
        self._tok = Tokenizer.from_file(os.path.join(model_dir, "tokenizer.json"))
        self._eos: List[int] = []
        cfg = os.path.join(model_dir, "tokenizer_config.json")
        if os.path.isfile(cfg):
            with open(cfg, "r", encoding="utf-8") as f:
                raw = json.load(f)
            eos = raw.get("eos_token")
            if isinstance(eos, dict):
                eos = eos.get("content")
            if isinstance(eos, str):
                tid = self._tok.token_to_id(eos)
                if tid is not None:
                    self._eos.append(tid)

    def encode(self, text: str) -> List[int]:
        return self._tok.encode(text, add_special_tokens=False).ids

    def decode(self, ids: Sequence[int]) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=True)

    def apply_chat_template(self, messages) -> str:
        return _chatml(messages)

    def eos_token_ids(self) -> List[int]:
        return list(self._eos)


def load_tokenizer(model_dir, vocab_size: int):
    """`model_dir` may be None (a model built in memory): the byte tokenizer."""
    if model_dir and os.path.isfile(os.path.join(model_dir, "tokenizer.json")):
        return FileTokenizer(model_dir)
    return ByteTokenizer(vocab_size)
