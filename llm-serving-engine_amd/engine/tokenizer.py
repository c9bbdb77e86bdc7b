"""Tokenizers: text <-> token ids (reference `tokenizer.py:6-45`)."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Protocol


class Tokenizer(Protocol):
    eos_token_id: int
    vocab_size: int

    def encode(self, text: str) -> list[int]: ...

    def decode(self, token_ids: list[int]) -> str: ...


class ByteTokenizer:
    """UTF-8 bytes shifted past four reserved ids (pad 0, bos 1, eos 2, 3 unused):
    260 ids, no files needed (`tokenizer.py:15-29`)."""

    pad_token_id = 0
    bos_token_id = 1
    eos_token_id = 2
    reserved = 4
    vocab_size = 256 + reserved

    def encode(self, text: str) -> list[int]:
        return [value + self.reserved for value in text.encode("utf-8")]

    def decode(self, token_ids: list[int]) -> str:
        data = bytes(t - self.reserved for t in token_ids if self.reserved <= t < self.vocab_size)
        return data.decode("utf-8", errors="replace")


def folder_eos_token_ids(folder: str | Path) -> tuple[int, ...]:
    """The end-of-sequence ids a model folder names: `eos_token_id` (a number or a list) of its
    generation_config.json, else of its config.json; none if neither file has the key."""
    for name in ("generation_config.json", "config.json"):
        path = Path(folder) / name
        if not path.is_file():
            continue
        found = json.loads(path.read_text()).get("eos_token_id")
        if found is None:
            continue
        ids = found if isinstance(found, (list, tuple)) else [found]
        return tuple(int(token) for token in ids)
    return ()


class FileTokenizer:
    """The tokenizer.json of a model folder, through the `tokenizers` library
    (the reference goes through `transformers.AutoTokenizer`, `tokenizer.py:32-45`).
    `eos_token_id` is the folder's own (generation_config.json, else config.json) unless
    one is given; -1 where the folder names none."""

    def __init__(self, folder: str | Path, eos_token_id: int | None = None) -> None:
        try:
            from tokenizers import Tokenizer as Inner
        except ImportError as error:  # pragma: no cover
            raise ImportError("the tokenizers package is needed to read tokenizer.json") from error
        path = Path(folder) / "tokenizer.json"
        if not path.is_file():
            raise FileNotFoundError(f"no tokenizer.json under {folder}")
        self.inner = Inner.from_file(str(path))
        self.vocab_size = self.inner.get_vocab_size()
        if eos_token_id is None:
            named = folder_eos_token_ids(folder)
            eos_token_id = named[0] if named else -1
        self.eos_token_id = int(eos_token_id)

    def encode(self, text: str) -> list[int]:
        return list(self.inner.encode(text, add_special_tokens=False).ids)

    def decode(self, token_ids: list[int]) -> str:
        return self.inner.decode(list(token_ids), skip_special_tokens=True)
