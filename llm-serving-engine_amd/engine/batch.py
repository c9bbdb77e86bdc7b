"""The facts about one step that every part may read: which tokens run, at
which positions, for which request, and where their cache entries lie.

One step is a flat list of T tokens.  Request b contributes the consecutive
tokens [query_start[b], query_start[b+1]) at positions
[context_length[b] - count, context_length[b]): a portion of a prompt, a single
decoded token, anything between.  The reference passes the same facts per row
(`engine.py:303-315`, `kv_cache.py:208-247`); here they are per request, so a
kernel can treat a portion as a tile of queries rather than as unrelated rows.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import torch

from ..cache.cell import CacheCell  # noqa: F401  (parts and tests find it here too)


@dataclass(frozen=True)
class SequenceChunk:
    """Host-side record of one request's share of the step."""

    request_id: str
    slot: int  # the request's state slot and block-table row
    start: int  # position of its first token in this step
    count: int  # tokens in this step

    @property
    def context_length(self) -> int:
        return self.start + self.count


@dataclass
class GroupBatch:
    """Per cache group: where this step's tokens are written, and each request's pages."""

    page_size: int
    block_tables: torch.Tensor  # int32 [B, width]; -1 where no page is held
    slot_mapping: torch.Tensor  # int32 [T]: page * page_size + offset
    width: int


@dataclass
class StepBatch:
    num_tokens: int
    chunks: list[SequenceChunk]
    token_ids: torch.Tensor  # int32 [T]
    positions: torch.Tensor  # int32 [T]
    token_sequence: torch.Tensor  # int32 [T]: index b of the token's request in this step
    query_start: torch.Tensor  # int32 [B + 1]
    context_lengths: torch.Tensor  # int32 [B]: tokens cached after this step
    state_slots: torch.Tensor  # int32 [B]
    groups: list[GroupBatch]
    logit_rows: torch.Tensor  # int32 [R]: token rows whose logits are wanted
    num_logit_rows: int
    max_query_length: int
    max_context_length: int
    every_row_wanted: bool = False  # logit_rows is 0, 1, ..., T - 1 (a step of single tokens): nothing to gather
    # (tokens, requests) that the arrays are padded to when the step's kernels are captured into a graph for
    # replay with other steps of the same padded shape: the arrays hold rows beyond the real ones (tokens that
    # are stored nowhere and whose results nobody reads, requests without tokens), `chunks` only the real requests.
    padded_to: tuple[int, int] | None = None
    # Kernel libraries may keep here what they derive from the step's shape on the host (work
    # lists: built once, used by every layer, and still valid when a captured step is replayed) ...
    scratch: dict[str, Any] = field(default_factory=dict)
    # ... and here what a kernel computes from the step's values (rotary angles): valid for one
    # forward pass only, so a captured step records the kernel that fills it.
    computed: dict[str, Any] = field(default_factory=dict)

    @property
    def num_sequences(self) -> int:
        return len(self.chunks)
