"""Dependency-free UTF-8 byte tokenizer for demos with random-weight models
(src/tokenvault/model_loader.py:127-139): bos 256, eos 257, vocabulary 258."""

from __future__ import annotations


class ByteTokenizer:
    def __init__(self) -> None:
        self.bos_token_id = 256
        self.eos_token_id = 257
        self.vocab_size = 258

    def encode(self, text: str) -> list[int]:
        return [self.bos_token_id, *text.encode("utf-8")]

    def decode(self, token_ids: list[int]) -> str:
        return bytes(t for t in token_ids if 0 <= t < 256).decode("utf-8", errors="replace")
