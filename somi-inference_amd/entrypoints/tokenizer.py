"""Optional text front: a thin wrapper over a tokenizer library.

Reference: ``Tokenizer`` (somi_inference/tokenizer.py:42-76): encode without
special tokens, decode skipping them, ``eos_token_id`` must exist.  Token ids are
this engine's contract; text works when the model folder carries tokenizer files.
"""

from __future__ import annotations

import os

_TOKENIZER_FILES = ("tokenizer.json", "tokenizer_config.json", "vocab.json", "tokenizer.model")


def has_tokenizer_files(model_dir: str) -> bool:
    return any(os.path.isfile(os.path.join(model_dir, name)) for name in _TOKENIZER_FILES)


class Tokenizer:
    def __init__(self, model_name: str) -> None:
        from transformers import AutoTokenizer   # a tokenizer library, no model code
        self.hf_tokenizer = AutoTokenizer.from_pretrained(model_name, local_files_only=True)
        if self.hf_tokenizer.eos_token_id is None:
            raise ValueError("Tokenizer must define eos_token_id")
        self.eos_token_id = int(self.hf_tokenizer.eos_token_id)

    def encode(self, text: str) -> list[int]:
        return list(self.hf_tokenizer.encode(text, add_special_tokens=False))

    def batch_encode(self, texts: list[str]) -> list[list[int]]:
        return [list(ids) for ids in self.hf_tokenizer(texts, add_special_tokens=False)["input_ids"]]

    def decode(self, token_ids: list[int]) -> str:
        return self.hf_tokenizer.decode(token_ids, skip_special_tokens=True)

    def batch_decode(self, token_ids_list: list[list[int]]) -> list[str]:
        return list(self.hf_tokenizer.batch_decode(token_ids_list, skip_special_tokens=True))
