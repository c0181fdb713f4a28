"""Chat templates and the text of a stream (no GPU).  The tokenizer of these tests is made in
memory: byte-level, one token a byte, so that a character outside ASCII spans several tokens."""
import json

import pytest

from xinfer_amd.config.engine_config import Message
from xinfer_amd.engine.tokenizer import (ByteTokenizer, FileTokenizer, IncrementalText, load_tokenizer,
                                         render_chat_template)
from xinfer_amd.models import family_of


def _byte_level_folder(tmp_path, config=None):
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    vocab = {c: i for i, c in enumerate(sorted(pre_tokenizers.ByteLevel.alphabet()))}
    vocab["<|end|>"] = len(vocab)
    tok = Tokenizer(models.BPE(vocab=vocab, merges=[]))
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    tok.save(str(tmp_path / "tokenizer.json"))
    if config is not None:
        (tmp_path / "tokenizer_config.json").write_text(json.dumps(config))
    return str(tmp_path)


def test_stream_text_waits_for_whole_characters(tmp_path):
    tok = FileTokenizer(_byte_level_folder(tmp_path))
    text = "héllo wörld ✓ ok"
    ids = tok.encode(text)
    assert len(ids) > len(text)                                 # é, ö and ✓ span two and three tokens
    inc = IncrementalText(tok)
    pieces = [inc.add(ids[:n]) for n in range(1, len(ids) + 1)]
    assert "".join(pieces) == text
    assert all("�" not in p for p in pieces)
    assert pieces[1] == "" and pieces[2] == "é"                 # the first byte of é waits for the second
    assert [p for p in pieces if p][-4:] == ["✓", " ", "o", "k"]
    # token by token, each decoded alone, breaks the characters: the case this class is for
    assert "�" in "".join(tok.decode([i]) for i in ids)


def test_stream_text_held_back_is_flushed_at_the_end(tmp_path):
    """A request cut inside a character that spans several tokens (by max_tokens, say): the pieces
    and what `finish` hands on are together the text of all tokens, as one decode gives it."""
    tok = FileTokenizer(_byte_level_folder(tmp_path))
    for text, cut in (("a ✓", 1), ("wörld", 4), ("ok", 0), ("é", 1)):
        ids = tok.encode(text)
        ids = ids[:len(ids) - cut]
        inc = IncrementalText(tok)
        pieces = [inc.add(ids[:n]) for n in range(1, len(ids) + 1)]
        rest = inc.finish(ids)
        assert "".join(pieces) + rest == tok.decode(ids), (text, cut)
        assert (rest != "") == (cut > 0) and inc.finish(ids) == ""


def test_chat_template_of_the_folder_is_rendered(tmp_path):
    """tokenizer_config.json's chat_template is rendered with the reference's variables
    (/root/reference/src/utils/chat_template.rs:459-472)."""
    template = ("{{ bos_token }}{% for m in messages %}[{{ m.role }}]{{ m.content }}{{ eos_token }}{% endfor %}"
                "{% if add_generation_prompt %}[assistant]{% if enable_thinking %}<think>{% endif %}{% endif %}")
    d = _byte_level_folder(tmp_path, {"chat_template": template, "bos_token": "<s>",
                                      "eos_token": {"content": "<|end|>"}})
    tok = load_tokenizer(d, 300, default_chat_template="never used")
    assert isinstance(tok, FileTokenizer) and tok.eos_token_ids() == [256]
    got = tok.apply_chat_template([Message("system", "be brief"), Message("user", "hi")])
    assert got == "<s>[system]be brief<|end|>[user]hi<|end|>[assistant]<think>"


def test_family_default_template_is_chatml(tmp_path):
    """A folder without a template gets its family's default: ChatML for Qwen3."""
    d = _byte_level_folder(tmp_path)
    tok = load_tokenizer(d, 300, family_of("Qwen3ForCausalLM").chat_template)
    got = tok.apply_chat_template([Message("system", "s"), Message("user", "u")])
    assert got == "<|im_start|>system\ns<|im_end|>\n<|im_start|>user\nu<|im_end|>\n<|im_start|>assistant\n"
    with pytest.raises(ValueError, match="no chat template"):
        load_tokenizer(d, 300, None).apply_chat_template([Message("user", "u")])
    assert isinstance(load_tokenizer(None, 300), ByteTokenizer)


def test_template_runs_in_a_sandbox_and_can_refuse():
    with pytest.raises(ValueError, match="chat template: roles must alternate"):
        render_chat_template("{{ raise_exception('roles must alternate') }}", [Message("user", "u")])
    from jinja2.exceptions import SecurityError
    with pytest.raises(SecurityError):
        render_chat_template("{{ messages.__class__.__mro__ }}", [Message("user", "u")])
