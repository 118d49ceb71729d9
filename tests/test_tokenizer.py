"""The optional text front over a tokenizer file made here (no downloaded vocabulary)."""

import json

import pytest

from somi_inference_amd.entrypoints.tokenizer import Tokenizer, has_tokenizer_files


def write_tokenizer(folder, eos_config=None):
    from tokenizers import Tokenizer as Codec
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    vocab = {"<unk>": 0, "<eos>": 1, "the": 2, "cat": 3, "sat": 4}
    codec = Codec(WordLevel(vocab, unk_token="<unk>"))
    codec.pre_tokenizer = Whitespace()
    codec.add_special_tokens(["<eos>"])
    codec.save(str(folder / "tokenizer.json"))
    if eos_config is not None:
        name, content = eos_config
        (folder / name).write_text(json.dumps(content))


def test_text_is_encoded_without_special_tokens_and_decoded_skipping_them(tmp_path):
    # the rules of the reference's wrapper: somi_inference/tokenizer.py:55-76
    assert not has_tokenizer_files(str(tmp_path))
    write_tokenizer(tmp_path, ("tokenizer_config.json", {"eos_token": "<eos>"}))
    assert has_tokenizer_files(str(tmp_path))
    tok = Tokenizer(str(tmp_path))
    assert tok.eos_token_id == 1
    assert tok.encode("the cat sat") == [2, 3, 4]
    assert tok.decode([2, 3, 1]) == "the cat"


def test_end_of_sequence_id_from_the_folders_other_files_or_an_error(tmp_path):
    a, b, c = tmp_path / "a", tmp_path / "b", tmp_path / "c"
    for folder in (a, b, c):
        folder.mkdir()
    write_tokenizer(a, ("tokenizer_config.json", {"eos_token": {"content": "<eos>"}}))
    assert Tokenizer(str(a)).eos_token_id == 1
    write_tokenizer(b, ("generation_config.json", {"eos_token_id": [4, 1]}))
    assert Tokenizer(str(b)).eos_token_id == 4
    write_tokenizer(c)
    with pytest.raises(ValueError, match="eos_token_id"):       # somi_inference/tokenizer.py:52-53
        Tokenizer(str(c))
