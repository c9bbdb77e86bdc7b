"""Tokenizers: text <-> token ids (reference `tokenizer.py:6-45`)."""

from __future__ import annotations

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


class FileTokenizer:
    """The tokenizer.json of a model folder, through the `tokenizers` library
    (the reference goes through `transformers.AutoTokenizer`, `tokenizer.py:32-45`)."""

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
        self.eos_token_id = -1 if eos_token_id is None else int(eos_token_id)

    def encode(self, text: str) -> list[int]:
        return list(self.inner.encode(text, add_special_tokens=False).ids)

    def decode(self, token_ids: list[int]) -> str:
        return self.inner.decode(list(token_ids), skip_special_tokens=True)
