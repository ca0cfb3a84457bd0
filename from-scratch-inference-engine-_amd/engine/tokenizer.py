"""Thin wrapper over a ``tokenizer.json`` (python/engine/tokenizer.py:14-32 in the reference)."""

from __future__ import annotations

from pathlib import Path
from typing import List


class EngineTokenizer:
    def __init__(self, tokenizer):
        self._tok = tokenizer

    @classmethod
    def from_model_dir(cls, model_dir) -> "EngineTokenizer":
        path = Path(model_dir) / "tokenizer.json"
        if not path.is_file():
            raise FileNotFoundError(f"no tokenizer.json in {model_dir}: pass token ids (generate_ids) instead of text")
        from tokenizers import Tokenizer

        return cls(Tokenizer.from_file(str(path)))

    def encode(self, text: str) -> List[int]:
        return list(self._tok.encode(text).ids)

    def decode(self, ids: List[int]) -> str:
        return self._tok.decode(list(ids))
