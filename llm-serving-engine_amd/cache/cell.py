"""What one run of a layer sees of the cache."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch


@dataclass
class CacheCell:
    """What one run of a layer sees of the cache.

    For a paged need: `keys` is [pages, kv_heads, page_size, head_dim], `values`
    is stored transposed, [pages, kv_heads, head_dim, page_size] (attention
    sums over keys, and the matrix cores want the summed index contiguous), and
    `group` indexes `StepBatch.groups`.  For a fixed state:
    `state` is [slots, *shape] float32, indexed by `StepBatch.state_slots`.
    `writable` is False when the run reads a cell that another run owns.
    """

    need: Any
    writable: bool = True
    group: int = -1
    keys: torch.Tensor | None = None
    values: torch.Tensor | None = None
    state: torch.Tensor | None = None
