"""A tokenizer that needs no files: one token per UTF-8 byte, for trying a random-weight model
with text.  Ids 0..255 are the bytes; 256 begins a text and 257 ends one, as in the reference's
``ByteTokenizer`` (src/tokenvault/model_loader.py:127-139), so a model needs a vocabulary of at
least 258."""

from __future__ import annotations

from typing import Iterable

BYTES = 256


class ByteTokenizer:
    bos_token_id = BYTES
    eos_token_id = BYTES + 1
    vocab_size = BYTES + 2

    def __init__(self, add_bos: bool = True) -> None:
        self.add_bos = add_bos

    def encode(self, text: str) -> list[int]:
        ids = list(text.encode("utf-8"))
        return [self.bos_token_id] + ids if self.add_bos else ids

    def decode(self, token_ids: Iterable[int]) -> str:
        """Special ids are dropped; bytes that do not form UTF-8 become U+FFFD."""
        data = bytearray(t for t in token_ids if 0 <= t < BYTES)
        return data.decode("utf-8", errors="replace")
