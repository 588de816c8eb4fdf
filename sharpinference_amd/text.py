"""Text at the edges of the command line: a model folder's ``tokenizer.json``, if it has one.

The engine itself runs on token ids only.  The reference reads its tokenizer from the GGUF
file's metadata (reference: src/SharpInference.Core/GgufTokenizer.cs:160-360); a safetensors
folder carries a ``tokenizer.json`` instead, which the ``tokenizers`` package reads.  A folder
without one is used with token ids.
"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence


def format_llama4_chat(user: str, system: Optional[str] = None) -> str:
    """One user turn in the Llama 4 chat form the reference falls back to when a model carries no
    template of its own (reference: src/SharpInference.Cli/RunCommand.cs:2588-2596): begin of
    text, then per message a header naming the role, a blank line, the text and an end-of-turn
    mark; it ends with the assistant's header, which the model continues."""
    out = "<|begin_of_text|>"
    if system is not None:
        out += f"<|header_start|>system<|header_end|>\n\n{system}<|eot|>"
    out += f"<|header_start|>user<|header_end|>\n\n{user}<|eot|>"
    return out + "<|header_start|>assistant<|header_end|>\n\n"


class TextCodec:
    """Encodes a prompt and decodes generated ids as they come."""

    def __init__(self, tokenizer, bos_token_id: Optional[int] = None):
        self._tok = tokenizer
        self.bos_token_id = bos_token_id

    @classmethod
    def from_folder(cls, model_dir: str, bos_token_id: Optional[int] = None) -> Optional["TextCodec"]:
        path = os.path.join(model_dir, "tokenizer.json")
        if not os.path.isfile(path):
            return None
        try:
            from tokenizers import Tokenizer
        except ImportError as e:  # pragma: no cover - the package is part of the environment
            raise RuntimeError(f"{path} needs the 'tokenizers' package: {e}") from None
        return cls(Tokenizer.from_file(path), bos_token_id)

    def encode(self, text: str) -> List[int]:
        """Token ids of a prompt; the configuration's begin-of-text token leads it once
        (whether or not the tokenizer's own post-processing adds it)."""
        ids = list(self._tok.encode(text).ids)
        if self.bos_token_id is not None and (not ids or ids[0] != self.bos_token_id):
            ids.insert(0, self.bos_token_id)
        return ids

    def knows_chat_marks(self) -> bool:
        """Does the vocabulary hold the marks of the Llama 4 chat form as single tokens?"""
        return all(self._tok.token_to_id(t) is not None for t in ("<|header_start|>", "<|header_end|>", "<|eot|>"))

    def encode_chat(self, user: str, system: Optional[str] = None) -> List[int]:
        """Token ids of one user turn (and a system message) in the chat form; the form's own
        begin-of-text mark is the only one."""
        ids = list(self._tok.encode(format_llama4_chat(user, system), add_special_tokens=False).ids)
        return ids

    def decode(self, ids: Sequence[int]) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=True)

    def streamer(self) -> "TextStreamer":
        return TextStreamer(self)


class TextStreamer:
    """Turns ids that arrive one by one into pieces of text: a piece is held back while the
    ids so far end inside a character (the decoder then shows U+FFFD)."""

    def __init__(self, codec: TextCodec):
        self._codec = codec
        self._ids: List[int] = []
        self._shown = 0

    def push(self, token_id: int) -> str:
        self._ids.append(int(token_id))
        text = self._codec.decode(self._ids)
        if text.endswith("�"):
            return ""
        piece, self._shown = text[self._shown:], len(text)
        return piece

    def flush(self) -> str:
        text = self._codec.decode(self._ids)
        piece, self._shown = text[self._shown:], len(text)
        return piece
