"""Optional text front-end: a thin wrapper over a model folder's ``tokenizer.json``.

The engine's interface is token ids.  Where a folder ships a tokenizer file this wrapper gives
``encode(text, add_bos)`` / ``decode(ids, skip_special)`` as the reference's does
(``tokenizer.py:74-101``); it uses the ``tokenizers`` package only (no model code, no network).
"""

from __future__ import annotations

from pathlib import Path
from typing import List, Optional, Sequence


class Tokenizer:
    def __init__(self, tokenizer_file, bos_id: Optional[int] = None, eos_id: Optional[int] = None):
        from tokenizers import Tokenizer as _Fast

        self._tok = _Fast.from_file(str(tokenizer_file))
        self.bos_id = bos_id
        self.eos_id = eos_id

    @classmethod
    def from_folder(cls, folder, bos_id: Optional[int] = None, eos_id: Optional[int] = None) -> "Tokenizer":
        path = Path(folder) / "tokenizer.json"
        if not path.is_file():
            raise FileNotFoundError(f"{folder} has no tokenizer.json; give token ids instead of text")
        return cls(path, bos_id, eos_id)

    def encode(self, text: str, add_bos: bool = True) -> List[int]:
        ids = self._tok.encode(text, add_special_tokens=False).ids
        if add_bos and self.bos_id is not None:
            ids = [self.bos_id] + ids
        return ids

    def decode(self, ids: Sequence[int], skip_special: bool = True) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=skip_special)
