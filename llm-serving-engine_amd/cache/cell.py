"""What one run of a layer sees of the cache."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch


KEY_PIECE = 8  # elements of a key that stay together in a page (csrc/common.h has the same number)


def key_piece_width(head_dim: int) -> int:
    """A key is kept in pieces of KEY_PIECE elements; a head size that is no multiple of it in one piece."""
    return KEY_PIECE if head_dim % KEY_PIECE == 0 else head_dim


@dataclass
class CacheCell:
    """What one run of a layer sees of the cache.

    For a paged need: `keys` is [pages, kv_heads, head_dim / w, page_size, w] with w =
    `key_piece_width(head_dim)`: a key lies in pieces of w elements, the same piece of all
    the keys of a page side by side (the matrix cores take keys as rows, a lane holding one
    piece of one key and its neighbours that piece of the next keys, and neighbouring lanes
    should read neighbouring bytes).  `values` is stored transposed, [pages, kv_heads,
    head_dim, page_size] (attention sums over keys, and the matrix cores want the summed
    index contiguous).  `group` indexes `StepBatch.groups`.  For a fixed state: `state` is
    [slots, *shape] float32, indexed by `StepBatch.state_slots`.  `writable` is False when
    the run reads a cell that another run owns.
    """

    need: Any
    writable: bool = True
    group: int = -1
    keys: torch.Tensor | None = None
    values: torch.Tensor | None = None
    state: torch.Tensor | None = None

    def key_rows(self, pages: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
        """The keys at (pages[i], offsets[i]) as whole rows, [n, kv_heads, head_dim]."""
        picked = self.keys[pages, :, :, offsets]  # [n, kv_heads, pieces, w]
        return picked.reshape(picked.shape[0], picked.shape[1], -1)

    def put_key_rows(self, pages: torch.Tensor, offsets: torch.Tensor, rows: torch.Tensor) -> None:
        """Writes whole rows [n, kv_heads, head_dim] as the keys at (pages[i], offsets[i])."""
        pieces, width = self.keys.shape[2], self.keys.shape[4]
        self.keys[pages, :, :, offsets] = rows.reshape(rows.shape[0], rows.shape[1], pieces, width).to(self.keys.dtype)
