"""Tokenizers for the command line.  ``CharTokenizer`` is the reference's
(fms/utils/tokenizers.py:97-143): a character is its code point, 256 tokens,
bos 2, eos 3.  Files of other tokenizers are opened with the libraries that
read them, if those are installed."""

from __future__ import annotations

import os
from typing import List


class CharTokenizer:
    """A character is the token of its code point: 256 tokens, code points from 256 on become token 0;
    token 2 begins a text and token 3 ends it (the ASCII controls of those names)."""

    bos_token_id = 2
    eos_token_id = 3
    _SIZE = 256

    def vocab_size(self) -> int:
        return self._SIZE

    def encode(self, text: str) -> List[int]:
        return [code if code < self._SIZE else 0 for code in map(ord, text)]

    def decode(self, ids) -> str:
        return "".join(map(chr, map(int, ids)))

    # the reference's older four-call interface (tests/utils/test_generate.py uses it)
    def tokenize(self, text: str) -> List[str]:
        return [c for c in text]

    def convert_tokens_to_ids(self, tokens):
        if isinstance(tokens, str):  # one token gives one id, as the reference's other tokenizers do
            if len(tokens) != 1:
                raise RuntimeError(f"a token of the character tokenizer is one character, got {tokens!r}")
            return self.encode(tokens)[0]
        return [self.encode(t)[0] if len(t) == 1 else 0 for t in tokens]

    def convert_ids_to_tokens(self, ids) -> List[str]:
        return list(self.decode(ids))

    def convert_tokens_to_string(self, tokens) -> str:
        return "".join(tokens)


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
