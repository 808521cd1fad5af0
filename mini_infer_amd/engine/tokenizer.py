"""Optional text interface: a `tokenizer.json` in the model folder.

Token ids are the engine's primary interface.  The reference wraps the
transformers tokenizer (engine/tokenizer.py:50-186); here the small `tokenizers`
package reads `tokenizer.json` directly when both are there, and the end-of-sequence
id comes from config.json's `eos_token_id`.
"""

from __future__ import annotations

from pathlib import Path
from typing import Sequence


class Tokenizer:
    def __init__(self, path: Path) -> None:
        from tokenizers import Tokenizer as _Tokenizer

        self._tok = _Tokenizer.from_file(str(path))

    @classmethod
    def from_pretrained(cls, model_dir: str | Path) -> "Tokenizer | None":
        path = Path(model_dir) / "tokenizer.json"
        if not path.exists():
            return None
        try:
            return cls(path)
        except ImportError:
            return None

    def encode(self, text: str) -> list[int]:
        return list(self._tok.encode(text).ids)

    def decode(self, ids: Sequence[int]) -> str:
        return self._tok.decode(list(ids))
