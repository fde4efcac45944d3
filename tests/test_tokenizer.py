"""The two tokenizers behind the reference's protocol (src/tokenvault/model_loader.py:116-139)."""

import json

import pytest

from kvforge_amd.tokenizer import ByteTokenizer, FileTokenizer, tokenizer_for


def test_bytes_round_trip_and_special_ids():
    tok = ByteTokenizer()
    ids = tok.encode("héllo")
    assert ids[0] == tok.bos_token_id == 256 and tok.eos_token_id == 257 and tok.vocab_size == 258
    assert ids[1:] == list("héllo".encode("utf-8"))
    assert tok.decode(ids + [tok.eos_token_id]) == "héllo"
    assert ByteTokenizer(add_bos=False).encode("a") == [97]
    assert tok.decode([0xE9]) == "�"                     # half a character


def test_a_folder_with_tokenizer_json_brings_its_own(tmp_path):
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    from tokenizers.processors import TemplateProcessing
    vocab = {"<s>": 0, "</s>": 1, "<unk>": 2, "a": 3, "page": 4, "of": 5, "keys": 6}
    tok = tokenizers.Tokenizer(WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = Whitespace()
    tok.post_processor = TemplateProcessing(single="<s> $A", special_tokens=[("<s>", 0)])
    tok.add_special_tokens(["<s>", "</s>"])
    tok.save(str(tmp_path / "tokenizer.json"))
    (tmp_path / "config.json").write_text(json.dumps({"bos_token_id": 0, "eos_token_id": [1, 9]}))
    mine = tokenizer_for(str(tmp_path))
    assert isinstance(mine, FileTokenizer)
    assert (mine.bos_token_id, mine.eos_token_id, mine.vocab_size) == (0, 1, 7)
    ids = mine.encode("a page of keys and values")
    assert ids == [0, 3, 4, 5, 6, 2, 2]                        # begins as the file says; unknown words
    assert mine.decode(ids[:5] + [1]) == "a page of keys"      # special tokens are dropped


def test_without_tokenizer_json_text_goes_byte_by_byte(tmp_path):
    assert isinstance(tokenizer_for(str(tmp_path)), ByteTokenizer)
    assert isinstance(tokenizer_for(None), ByteTokenizer)
    with pytest.raises(FileNotFoundError):
        FileTokenizer(str(tmp_path))
