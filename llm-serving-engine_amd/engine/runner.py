"""The step function: one batch of (request, its next tokens) through the model.

`ModelRunner.step` is the only way tokens reach the model: generation, the
scheduler and trace replay all call it.  It reserves cache entries for exactly
the tokens it is given, runs them as one batch against what earlier steps left
in the cache, and returns the logits at the wanted places.  The reference's
counterpart is the second half of `LLMEngine._step` plus
`Transformer.forward_paged` (`engine.py:269-315`, `model.py:270-309`).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.manager import CacheManager, Reservation
from ..cache.pool import CacheFullError
from ..config.serving import CacheConfig
from ..parts.model import DecoderModel
from ..weights.loader import LoadedModel
from .batch import GroupBatch, SequenceChunk, StepBatch


@dataclass(frozen=True)
class StepEntry:
    """One request's share of a step: its next tokens and the places among them
    (0-based, within `tokens`) whose logits are wanted."""

    request_id: str
    tokens: tuple[int, ...] | list[int]
    want: tuple[int, ...] | list[int] = field(default_factory=tuple)


def build_step_batch(
    reservations: list[Reservation],
    entries: list[StepEntry],
    cache: CacheManager,
    device: torch.device,
) -> StepBatch:
    """All index arrays of a step, packed on the host and sent in one copy."""
    counts = np.array([r.count for r in reservations], dtype=np.int64)
    total = int(counts.sum())
    query_start = np.zeros(len(reservations) + 1, dtype=np.int32)
    query_start[1:] = np.cumsum(counts)
    token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
    positions = np.concatenate([np.arange(r.start, r.start + r.count, dtype=np.int32) for r in reservations])
    token_sequence = np.repeat(np.arange(len(reservations), dtype=np.int32), counts)
    context = np.array([r.start + r.count for r in reservations], dtype=np.int32)
    slots = np.array([r.slot for r in reservations], dtype=np.int32)
    rows = [query_start[b] + np.asarray(e.want, dtype=np.int32) for b, e in enumerate(entries)]
    logit_rows = np.concatenate(rows).astype(np.int32) if rows else np.zeros(0, np.int32)

    pieces = [token_ids, positions, token_sequence, query_start, context, slots, logit_rows]
    widths = []
    for index, group in enumerate(cache.groups):
        width = max(1, int(-(-int(context.max()) // cache.page_size)))
        widths.append(width)
        pieces.append(np.concatenate([r.slots[index] for r in reservations]))
        pieces.append(group.tables[slots, :width].reshape(-1))
    sizes = [piece.size for piece in pieces]
    packed = torch.from_numpy(np.concatenate(pieces).astype(np.int32, copy=False))
    on_device = packed.to(device)
    views = list(torch.split(on_device, sizes))
    groups = []
    for index in range(len(cache.groups)):
        mapping, tables = views[7 + 2 * index], views[8 + 2 * index]
        groups.append(
            GroupBatch(cache.page_size, tables.view(len(reservations), widths[index]), mapping, widths[index])
        )
    chunks = [SequenceChunk(r.request_id, r.slot, r.start, r.count) for r in reservations]
    return StepBatch(
        num_tokens=total,
        chunks=chunks,
        token_ids=views[0],
        positions=views[1],
        token_sequence=views[2],
        query_start=views[3],
        context_lengths=views[4],
        state_slots=views[5],
        groups=groups,
        logit_rows=views[6],
        num_logit_rows=int(logit_rows.size),
        max_query_length=int(counts.max()),
        max_context_length=int(context.max()),
    )


class ModelRunner:
    """A model, its cache and the step function over them."""

    def __init__(
        self,
        loaded: LoadedModel,
        kernels,
        cache_config: CacheConfig | None = None,
        *,
        max_sequence_length: int | None = None,
    ) -> None:
        self.loaded = loaded
        self.kernels = kernels
        self.spec = loaded.spec
        self.dtype = loaded.dtype
        self.device = torch.device(kernels.device)
        self.cache_config = cache_config or CacheConfig()
        if max_sequence_length is None:
            max_sequence_length = getattr(loaded.config, "max_position_embeddings", None)
        if max_sequence_length is None:
            raise ValueError("max_sequence_length is needed for a config without max_position_embeddings")
        tensors = {name: kernels.to_device(value) for name, value in loaded.tensors.items()}
        self.model = DecoderModel(loaded.spec, tensors, kernels)
        self.cache = CacheManager(
            loaded.spec,
            self.cache_config,
            max_sequence_length=max_sequence_length,
            dtype=loaded.dtype,
            device=self.device,
        )
        self.cells = self.cache.cells()
        self.vocab_size = loaded.spec.vocab_size

    def add_request(self, request_id: str) -> int:
        return self.cache.create(request_id)

    def end_request(self, request_id: str) -> None:
        self.cache.free(request_id)

    def has_request(self, request_id: str) -> bool:
        return request_id in self.cache.sequences

    def step(self, entries: list[StepEntry], *, create_missing: bool = False) -> torch.Tensor:
        """Runs the entries as one batch; returns float32 logits [wanted, vocab]
        in the order of the entries and of each entry's `want`.

        Nothing is reserved if the batch does not fit (`CacheFullError`)."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        for entry in entries:
            if entry.request_id in seen:
                raise ValueError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            if len(entry.tokens) == 0:
                raise ValueError(f"request {entry.request_id!r} brings no tokens")
            for place in entry.want:
                if not 0 <= place < len(entry.tokens):
                    raise ValueError(f"request {entry.request_id!r}: wanted place {place} is outside its tokens")
            for token in entry.tokens:
                if not 0 <= token < self.vocab_size:
                    raise ValueError(f"request {entry.request_id!r}: token {token} is outside the vocabulary")
        created = []
        try:
            for entry in entries:
                if not self.has_request(entry.request_id):
                    if not create_missing:
                        raise KeyError(f"unknown request {entry.request_id!r}")
                    self.add_request(entry.request_id)
                    created.append(entry.request_id)
            plan = [(entry.request_id, len(entry.tokens)) for entry in entries]
            if not self.cache.fits(plan):
                raise CacheFullError("the step's tokens do not fit the cache")
        except Exception:
            for request_id in created:
                self.end_request(request_id)
            raise
        reservations = [self.cache.reserve(request_id, count) for request_id, count in plan]
        batch = build_step_batch(reservations, entries, self.cache, self.device)
        return self.forward(batch)

    @torch.inference_mode()
    def forward(self, batch: StepBatch) -> torch.Tensor:
        if batch.num_logit_rows == 0:
            self.model.forward_without_logits(batch, self.cells)
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        return self.model.forward(batch, self.cells)
