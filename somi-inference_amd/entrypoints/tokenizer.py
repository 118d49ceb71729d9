"""Optional text front: token ids are this engine's contract; text works when the model folder carries a
``tokenizer.json``.

Reference: ``Tokenizer`` (somi_inference/tokenizer.py:42-76) wraps a library tokenizer: text is encoded
without special tokens, ids are decoded with special tokens skipped, and a tokenizer without an
end-of-sequence id is refused.  The same three rules hold here, over the ``tokenizers`` library's own file
format, with the end-of-sequence token looked up in the folder's ``tokenizer_config.json``,
``generation_config.json`` or ``config.json``.
"""

from __future__ import annotations

import json
import os

TOKENIZER_FILE = "tokenizer.json"


def has_tokenizer_files(model_dir: str) -> bool:
    return os.path.isfile(os.path.join(model_dir, TOKENIZER_FILE))


def _read_json(path: str) -> dict:
    if not os.path.isfile(path):
        return {}
    with open(path, "r", encoding="utf-8") as handle:
        loaded = json.load(handle)
    return loaded if isinstance(loaded, dict) else {}


class Tokenizer:
    def __init__(self, model_dir: str) -> None:
        from tokenizers import Tokenizer as Codec      # a tokenizer library: no model code
        self.codec = Codec.from_file(os.path.join(model_dir, TOKENIZER_FILE))
        self.eos_token_id = self._find_eos(model_dir)

    def _find_eos(self, model_dir: str) -> int:
        named = _read_json(os.path.join(model_dir, "tokenizer_config.json")).get("eos_token")
        if isinstance(named, dict):                     # {"content": "<|endoftext|>", ...}
            named = named.get("content")
        if isinstance(named, str) and self.codec.token_to_id(named) is not None:
            return int(self.codec.token_to_id(named))
        for name in ("generation_config.json", "config.json"):
            given = _read_json(os.path.join(model_dir, name)).get("eos_token_id")
            if isinstance(given, list) and given:
                given = given[0]
            if isinstance(given, int):
                return given
        raise ValueError("Tokenizer must define eos_token_id")       # the reference's message (tokenizer.py:52-53)

    def encode(self, text: str) -> list[int]:
        return list(self.codec.encode(text, add_special_tokens=False).ids)

    def decode(self, token_ids: list[int]) -> str:
        return self.codec.decode(list(token_ids), skip_special_tokens=True)
