"""What one run of a layer sees of the cache."""

from __future__ import annotations

from typing import Any

import torch

from ..parts.base import KEY_PIECE, VALUE_PIECE, key_piece_width, value_piece_width  # noqa: F401  (kernel libraries and tests find them here)


class CacheCell:
    """What one run of a layer sees of the cache, for one of its needs.

    For a paged need: `fields` holds, by the names the need gave in `page_fields`, the tensors
    [pages, *page shape] of this run, and `group` indexes `StepBatch.groups` (where the step's tokens
    go, and the requests' block tables).  For keys and values (`PagedKeyValue`): `keys` is [pages,
    kv_heads, head_dim / w, page_size, w] with w = `key_piece_width(head_dim)`, `values` is stored
    transposed in pieces of v = `value_piece_width(page_size)` keys, [pages, kv_heads, page_size / v, head_dim,
    v]; both are also attributes of the cell, and `key_rows` / `value_rows` give whole rows back.
    For a per-request need: `state` is [slots, *shape] float32, indexed by `StepBatch.state_slots`.
    `writable` is False when the run reads a cell that another run owns.
    """

    def __init__(
        self,
        need: Any,
        writable: bool = True,
        group: int = -1,
        keys: torch.Tensor | None = None,
        values: torch.Tensor | None = None,
        state: torch.Tensor | None = None,
        fields: dict[str, torch.Tensor] | None = None,
    ) -> None:
        self.need = need
        self.writable = writable
        self.group = group
        self.state = state
        self.fields: dict[str, torch.Tensor] = dict(fields or {})
        if keys is not None:
            self.fields["keys"] = keys
        if values is not None:
            self.fields["values"] = values

    @property
    def keys(self) -> torch.Tensor | None:
        return self.fields.get("keys")

    @keys.setter
    def keys(self, tensor: torch.Tensor) -> None:
        self.fields["keys"] = tensor

    @property
    def values(self) -> torch.Tensor | None:
        return self.fields.get("values")

    @values.setter
    def values(self, tensor: torch.Tensor) -> None:
        self.fields["values"] = tensor

    def key_rows(self, pages: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
        """The keys at (pages[i], offsets[i]) as whole rows, [n, kv_heads, head_dim]."""
        picked = self.keys[pages, :, :, offsets]  # [n, kv_heads, pieces, w]
        return picked.reshape(picked.shape[0], picked.shape[1], -1)

    def put_key_rows(self, pages: torch.Tensor, offsets: torch.Tensor, rows: torch.Tensor) -> None:
        """Writes whole rows [n, kv_heads, head_dim] as the keys at (pages[i], offsets[i])."""
        pieces, width = self.keys.shape[2], self.keys.shape[4]
        self.keys[pages, :, :, offsets] = rows.reshape(rows.shape[0], rows.shape[1], pieces, width).to(self.keys.dtype)

    def value_rows(self, pages: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
        """The values at (pages[i], offsets[i]) as whole rows, [n, kv_heads, head_dim]."""
        width = self.values.shape[4]
        return self.values[pages, :, offsets // width, :, offsets % width]

    def put_value_rows(self, pages: torch.Tensor, offsets: torch.Tensor, rows: torch.Tensor) -> None:
        """Writes whole rows [n, kv_heads, head_dim] as the values at (pages[i], offsets[i])."""
        width = self.values.shape[4]
        self.values[pages, :, offsets // width, :, offsets % width] = rows.to(self.values.dtype)
