"""Tokenizers for the command line.  ``CharTokenizer`` is the reference's
(fms/utils/tokenizers.py:97-143): a character is its code point, 256 tokens,
bos 2, eos 3.  Files of other tokenizers are opened with the libraries that
read them, if those are installed."""

from __future__ import annotations

import os
from typing import List, Optional


class CharTokenizer:
    """A character is the token of its code point: 256 tokens, code points from 256 on become token 0;
    token 2 begins a text and token 3 ends it (the ASCII controls of those names)."""

    bos_token_id = 2
    eos_token_id = 3
    _SIZE = 256

    def vocab_size(self) -> int:
        return self._SIZE

    def encode(self, text: str, add_special_tokens: bool = False) -> List[int]:
        ids = [code if code < self._SIZE else 0 for code in map(ord, text)]
        return [self.bos_token_id] + ids if add_special_tokens else ids

    def decode(self, ids, skip_special_tokens: bool = True) -> str:
        ids = [int(i) for i in ids]
        if skip_special_tokens:
            ids = [i for i in ids if i not in (self.bos_token_id, self.eos_token_id)]
        return "".join(map(chr, ids))

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
        return [chr(int(i)) for i in ids]

    def convert_tokens_to_string(self, tokens) -> str:
        return "".join(tokens)


class _FourCalls:
    """What the wrappers below share: the reference's interface (fms/utils/tokenizers.py:21-95) is encode/decode
    with the Hugging Face arguments, and the older four calls that its script still makes
    (scripts/inference.py:179-181, 232-234): text -> pieces -> ids and ids -> pieces -> text."""

    bos_token_id = 0
    eos_token_id = 0

    def encode(self, text: str, add_special_tokens: bool = False) -> List[int]:
        ids = self.convert_tokens_to_ids(self.tokenize(text))
        return [self.bos_token_id] + ids if add_special_tokens else ids

    def decode(self, ids, skip_special_tokens: bool = True) -> str:
        ids = [int(i) for i in ids]
        if skip_special_tokens:
            ids = [i for i in ids if i not in (self.bos_token_id, self.eos_token_id)]
        return self.convert_tokens_to_string(self.convert_ids_to_tokens(ids))


class _SentencePiece(_FourCalls):
    def __init__(self, path: str):
        import sentencepiece

        self.sp = sentencepiece.SentencePieceProcessor(model_file=path)
        self.bos_token_id, self.eos_token_id = self.sp.bos_id(), self.sp.eos_id()

    def tokenize(self, text: str) -> List[str]:
        return self.sp.encode(text, out_type=str)

    def convert_tokens_to_ids(self, tokens):
        return self.sp.piece_to_id(tokens)  # one piece gives one id, a list a list

    def convert_ids_to_tokens(self, ids) -> List[str]:
        return self.sp.id_to_piece([int(i) for i in ids])

    def convert_tokens_to_string(self, tokens) -> str:
        return self.sp.decode_pieces(list(tokens))

    def vocab_size(self):
        return self.sp.get_piece_size()


class _TokenizersJson(_FourCalls):
    def __init__(self, path: str):
        import tokenizers

        self.tk = tokenizers.Tokenizer.from_file(path)
        self.bos_token_id = self.tk.token_to_id("<s>") or self.tk.token_to_id("<|begin_of_text|>") or 0
        self.eos_token_id = self.tk.token_to_id("</s>") or self.tk.token_to_id("<|end_of_text|>") or 0

    def tokenize(self, text: str) -> List[str]:
        return self.tk.encode(text, add_special_tokens=False).tokens

    def convert_tokens_to_ids(self, tokens):
        if isinstance(tokens, str):
            return self.tk.token_to_id(tokens)
        return [self.tk.token_to_id(t) for t in tokens]

    def convert_ids_to_tokens(self, ids) -> List[str]:
        return [self.tk.id_to_token(int(i)) for i in ids]

    def convert_tokens_to_string(self, tokens) -> str:
        decoder = self.tk.decoder
        return decoder.decode(list(tokens)) if decoder is not None else " ".join(tokens)

    def decode(self, ids, skip_special_tokens: bool = True) -> str:
        return self.tk.decode([int(i) for i in ids], skip_special_tokens=bool(skip_special_tokens))

    def vocab_size(self):
        return self.tk.get_vocab_size()


def get_tokenizer(name: str, style: Optional[str] = None):
    """"char_tokenizer", a sentencepiece ``.model`` file, or a ``tokenizer.json`` (or its folder)
    (fms/utils/tokenizers.py:459-502).  style, as there: None (told from the name), "fms" (the character
    tokenizer), "sentencepiece" or "hf" (here: the folder's tokenizer.json, read with the `tokenizers` package)."""
    if style not in (None, "fms", "sentencepiece", "hf"):
        raise RuntimeError(f"unknown tokenizer style {style!r}: one of 'fms', 'sentencepiece', 'hf'")
    if name in ("char_tokenizer", "char") and style in (None, "fms"):
        return CharTokenizer()
    path = os.path.expanduser(name)
    if style == "sentencepiece" or (style is None and path.endswith(".model")):
        if not os.path.isfile(path):
            raise RuntimeError(f"Could not find SentencePiece model at '{name}'")
        return _SentencePiece(path)
    if os.path.isdir(path) and os.path.isfile(os.path.join(path, "tokenizer.json")):
        path = os.path.join(path, "tokenizer.json")
    if path.endswith(".json") and os.path.isfile(path):
        return _TokenizersJson(path)
    if style is None and os.path.isfile(path):
        return _SentencePiece(path)
    raise RuntimeError(f"Could not find tokenizer {name}")
