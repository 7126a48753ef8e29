"""The tokenizer of the command line: a tiktoken-style vocabulary file.

Behaviour of the reference's ``TikTokenizer`` (src/io/tokenizer.cpp:80-182): the file has
one ``base64(token bytes) id`` pair per line; encoding is greedy longest match over at
most 16 bytes (not BPE merges), a byte without a match is tried on its own and otherwise
skipped; ids 128000-128255 are the Llama 3 special tokens, 128000 begins a text and
128001 ends it (include/photon/io/tokenizer.hpp:31-93).
"""
from __future__ import annotations

import base64
import os
from typing import Dict, List

from .errors import ErrorCode, PhotonError

SPECIAL_FIRST, SPECIAL_LAST = 128000, 128255
MAX_MATCH_BYTES = 16


class TikTokenizer:
    def __init__(self, vocab: Dict[bytes, int]):
        if not vocab:
            raise PhotonError("empty vocabulary", ErrorCode.INVALID_ARGUMENT)
        self.vocab = vocab
        self.id_to_token: Dict[int, bytes] = {}
        for tok, i in vocab.items():
            self.id_to_token.setdefault(i, tok)
        for i in range(SPECIAL_FIRST, SPECIAL_LAST + 1):
            self.id_to_token.setdefault(i, f"<|reserved_special_token_{i - SPECIAL_FIRST}|>".encode())
        self.id_to_token[SPECIAL_FIRST] = b"<|begin_of_text|>"
        self.id_to_token[SPECIAL_FIRST + 1] = b"<|end_of_text|>"

    @classmethod
    def load(cls, path: str) -> "TikTokenizer":
        if not os.path.isfile(path):
            raise PhotonError(f"Tokenizer file not found: {path}", ErrorCode.FILE_NOT_FOUND)
        vocab: Dict[bytes, int] = {}
        with open(path, "r", encoding="utf-8", errors="replace") as f:
            for line in f:
                parts = line.rstrip("\n").split(" ")
                if len(parts) < 2:
                    continue
                try:
                    tok, i = base64.b64decode(parts[0]), int(parts[1])
                except ValueError:
                    continue
                vocab.setdefault(tok, i)
        if not vocab:
            raise PhotonError(f"Empty vocabulary loaded from: {path}", ErrorCode.INVALID_ARGUMENT)
        return cls(vocab)

    def vocab_size(self) -> int:
        return len(self.vocab)

    def bos_id(self) -> int:
        return SPECIAL_FIRST

    def eos_id(self) -> int:
        return SPECIAL_FIRST + 1

    def encode(self, text: str) -> List[int]:
        data = text.encode("utf-8")
        out, i = [], 0
        while i < len(data):
            for n in range(min(MAX_MATCH_BYTES, len(data) - i), 0, -1):
                tok = self.vocab.get(data[i:i + n])
                if tok is not None:
                    out.append(tok)
                    i += n
                    break
            else:
                i += 1   # a byte that is no token by itself is skipped
        return out

    def decode_token(self, token_id: int) -> str:
        return self.id_to_token.get(int(token_id), b"").decode("utf-8", "replace")

    def decode(self, tokens) -> str:
        return b"".join(self.id_to_token.get(int(t), b"") for t in tokens).decode("utf-8", "replace")
