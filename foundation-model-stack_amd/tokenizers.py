"""Tokenizers for the command line.  ``CharTokenizer`` is the reference's
(fms/utils/tokenizers.py:97-143): a character is its code point, 256 tokens,
bos 2, eos 3.  Files of other tokenizers are opened with the libraries that
read them, if those are installed."""

from __future__ import annotations

import os
from typing import List


class CharTokenizer:
    bos_token_id = 2
    eos_token_id = 3

    def tokenize(self, text: str) -> List[str]:
        return list(text)

    def convert_tokens_to_ids(self, tokens) -> List[int]:
        if isinstance(tokens, str):
            if len(tokens) != 1:
                raise RuntimeError("Only single character str tokens can be converted using the CharTokenizer.")
            return ord(tokens) if ord(tokens) < 256 else 0
        return [ord(t) if len(t) == 1 and ord(t) < 256 else 0 for t in tokens]

    def convert_ids_to_tokens(self, ids) -> List[str]:
        return [chr(int(i)) for i in ids]

    def convert_tokens_to_string(self, tokens: List[str]) -> str:
        return "".join(tokens)

    def encode(self, text: str) -> List[int]:
        return self.convert_tokens_to_ids(self.tokenize(text))

    def decode(self, ids) -> str:
        return self.convert_tokens_to_string(self.convert_ids_to_tokens(ids))

    def vocab_size(self) -> int:
        return 256


class _SentencePiece:
    def __init__(self, path: str):
        import sentencepiece

        self.sp = sentencepiece.SentencePieceProcessor(model_file=path)
        self.bos_token_id, self.eos_token_id = self.sp.bos_id(), self.sp.eos_id()

    def encode(self, text):
        return self.sp.encode(text)

    def decode(self, ids):
        return self.sp.decode([int(i) for i in ids])

    def vocab_size(self):
        return self.sp.get_piece_size()


class _TokenizersJson:
    def __init__(self, path: str):
        import tokenizers

        self.tk = tokenizers.Tokenizer.from_file(path)
        self.bos_token_id = self.tk.token_to_id("<s>") or self.tk.token_to_id("<|begin_of_text|>") or 0
        self.eos_token_id = self.tk.token_to_id("</s>") or self.tk.token_to_id("<|end_of_text|>") or 0

    def encode(self, text):
        return self.tk.encode(text, add_special_tokens=False).ids

    def decode(self, ids):
        return self.tk.decode([int(i) for i in ids])

    def vocab_size(self):
        return self.tk.get_vocab_size()


def get_tokenizer(name: str):
    """"char_tokenizer", a sentencepiece ``.model`` file, or a ``tokenizer.json`` (or its folder)
    (fms/utils/tokenizers.py:459-502)."""
    if name in ("char_tokenizer", "char"):
        return CharTokenizer()
    path = os.path.expanduser(name)
    if os.path.isdir(path) and os.path.isfile(os.path.join(path, "tokenizer.json")):
        path = os.path.join(path, "tokenizer.json")
    if path.endswith(".json") and os.path.isfile(path):
        return _TokenizersJson(path)
    if os.path.isfile(path):
        return _SentencePiece(path)
    raise RuntimeError(f"Could not find tokenizer {name}")
