"""Text in and out: tokenizer and chat template of a model folder.

The engine itself only sees token ids.  A folder with ``tokenizer.json`` is read with
the ``tokenizers`` package; a folder without one (random weights) gets a byte
tokenizer, ids = bytes, so that the command line works end to end.  The chat template
is the Jinja template of ``tokenizer_config.json`` with the reference's arguments
``messages, bos_token, eos_token, add_generation_prompt``
(llama.cu/src/model/chat_template.rs:85-113; its ``.strip()`` extension, :118-130, is a
string method that Jinja in Python has by itself).
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence


class ByteTokenizer:
    """ids = the bytes of the UTF-8 text (needs a vocabulary of at least 256)."""

    def __init__(self, vocab_size: int):
        if vocab_size < 256:
            raise ValueError(f"the byte tokenizer needs a vocabulary of at least 256, the model has {vocab_size}")

    def encode(self, text: str) -> List[int]:
        return list(text.encode("utf-8"))

    def decode(self, ids: Sequence[int]) -> str:
        return bytes(i for i in ids if 0 <= i < 256).decode("utf-8", errors="replace")


class FileTokenizer:
    def __init__(self, path: str):
        from tokenizers import Tokenizer
        self.tok = Tokenizer.from_file(path)

    def encode(self, text: str) -> List[int]:
        return list(self.tok.encode(text, add_special_tokens=False).ids)

    def decode(self, ids: Sequence[int]) -> str:
        return self.tok.decode(list(ids), skip_special_tokens=False)


def load_tokenizer(folder: str, vocab_size: int):
    path = os.path.join(folder, "tokenizer.json")
    return FileTokenizer(path) if os.path.isfile(path) else ByteTokenizer(vocab_size)


class StreamDecoder:
    """Turns tokens into text piece by piece; bytes of a character that is not yet whole
    are held back (the reference's ``TextBuf``, llama.cu/xtask/src/generate.rs:44,56)."""

    # how many tokens before the pending ones are decoded along with them: a tokenizer may render a token
    # differently after another (a leading space), so a piece is what a short context adds to its rendering
    CONTEXT = 8

    def __init__(self, tokenizer):
        self.tokenizer = tokenizer
        self.ids: List[int] = []
        self.done = 0                  # tokens whose text has been handed out

    def push(self, token: int) -> str:
        """The text that ``token`` completes ("" while a character's bytes are not all there).  Only the last few
        tokens are decoded, not the whole sequence so far."""
        self.ids.append(token)
        start = max(self.done - self.CONTEXT, 0)
        before = self.tokenizer.decode(self.ids[start:self.done])
        text = self.tokenizer.decode(self.ids[start:])
        if text.endswith("�") and len(self.ids) - self.done < 8:
            return ""
        self.done = len(self.ids)
        return text[len(before):] if text.startswith(before) else text


DEFAULT_TEMPLATE = ("{% for message in messages %}{{ message['role'] + ': ' + message['content'].strip() + '\\n' }}"
                    "{% endfor %}{% if add_generation_prompt %}{{ 'assistant: ' }}{% endif %}")


class ChatTemplate:
    def __init__(self, template: str, bos_token: str = "", eos_token: str = ""):
        import jinja2
        self.template = jinja2.Environment().from_string(template)
        self.bos, self.eos = bos_token, eos_token

    def render(self, messages: Sequence[Dict[str, str]], add_generation_prompt: bool = True) -> str:
        return self.template.render(messages=list(messages), bos_token=self.bos, eos_token=self.eos,
                                    add_generation_prompt=add_generation_prompt)


def _token_text(v) -> str:
    if isinstance(v, dict):
        return v.get("content", "")
    return v or ""


def load_chat_template(folder: str) -> ChatTemplate:
    path = os.path.join(folder, "tokenizer_config.json")
    if os.path.isfile(path):
        with open(path) as f:
            cfg = json.load(f)
        if cfg.get("chat_template"):
            return ChatTemplate(cfg["chat_template"], _token_text(cfg.get("bos_token")), _token_text(cfg.get("eos_token")))
    return ChatTemplate(DEFAULT_TEMPLATE)


def user(content: str) -> Dict[str, str]:
    return {"role": "user", "content": content}
