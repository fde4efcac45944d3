"""Text to token ids and back, behind the reference's tokenizer protocol
(src/tokenvault/model_loader.py:116-122: ``encode``, ``decode``, ``bos_token_id``,
``eos_token_id``).

``ByteTokenizer`` needs no files: one token per UTF-8 byte, for trying a random-weight model
with text.  Ids 0..255 are the bytes; 256 begins a text and 257 ends one, as in the reference's
``ByteTokenizer`` (src/tokenvault/model_loader.py:127-139), so a model needs a vocabulary of at
least 258.

``FileTokenizer`` reads the ``tokenizer.json`` that a checkpoint folder brings, where the
reference wraps the checkpoint's own tokenizer (scripts/serve.py:68)."""

from __future__ import annotations

import json
import os
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


class FileTokenizer:
    """The tokenizer a model folder describes in ``tokenizer.json``, read with the ``tokenizers``
    package.  What begins and ends a text comes from the folder's ``config.json``
    (``bos_token_id``, ``eos_token_id``; the first of a list); whether a text gets its beginning
    added is what the file's own post-processing says."""

    def __init__(self, folder: str) -> None:
        path = os.path.join(folder, "tokenizer.json")
        if not os.path.isfile(path):
            raise FileNotFoundError(f"no tokenizer.json in {folder}")
        try:
            from tokenizers import Tokenizer
        except ImportError as e:
            raise ImportError("reading tokenizer.json needs the `tokenizers` package") from e
        self._tok = Tokenizer.from_file(path)
        self.vocab_size = self._tok.get_vocab_size()
        self.bos_token_id = self.eos_token_id = None
        cfg_path = os.path.join(folder, "config.json")
        if os.path.isfile(cfg_path):
            with open(cfg_path) as f:
                cfg = json.load(f)
            self.bos_token_id, self.eos_token_id = (self._first(cfg.get(k)) for k in ("bos_token_id", "eos_token_id"))

    @staticmethod
    def _first(v):
        if isinstance(v, (list, tuple)):
            v = v[0] if v else None
        return None if v is None else int(v)

    def encode(self, text: str) -> list[int]:
        return list(self._tok.encode(text).ids)

    def decode(self, token_ids: Iterable[int]) -> str:
        return self._tok.decode([int(t) for t in token_ids], skip_special_tokens=True)


def tokenizer_for(folder: str | None):
    """The folder's own tokenizer if it brings one, else bytes."""
    if folder and os.path.isfile(os.path.join(folder, "tokenizer.json")):
        return FileTokenizer(folder)
    return ByteTokenizer()
