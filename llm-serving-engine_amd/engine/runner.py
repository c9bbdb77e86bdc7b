"""The step function: one batch of (request, its next tokens) through the model.

`ModelRunner.step` is the only way tokens reach the model: generation, the
scheduler and trace replay all call it.  It reserves cache entries for exactly
the tokens it is given, runs them as one batch against what earlier steps left
in the cache, and returns the logits at the wanted places.  The reference's
counterpart is the second half of `LLMEngine._step` plus
`Transformer.forward_paged` (`engine.py:269-315`, `model.py:270-309`).
"""

from __future__ import annotations

import contextlib
import time
from dataclasses import dataclass, field
from typing import Any

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


def _pack_step(
    reservations: list[Reservation],
    entries: list[StepEntry],
    cache: CacheManager,
    *,
    pad_to: int | None = None,
    width: int | None = None,
    pad_tokens_to: int | None = None,
    pad_rows_to: int | None = None,
) -> tuple[np.ndarray, list[int], list[int], dict]:
    """The step's index arrays as one int32 array: token ids, positions, request index per
    token, query starts, context lengths, state slots, wanted rows, then per cache group the
    slot of every token and the requests' block-table rows.  Padding, for a captured graph: with
    `pad_to`, requests are padded to that many; a padding request brings one token, or, with
    `pad_tokens_to`, the first of them brings all the tokens that are missing to that count and the
    others none.  Padding tokens are stored nowhere and read page 0.  `pad_rows_to` pads the wanted
    rows (with row 0); without it a padded step wants every request's row."""
    counts = np.array([r.count for r in reservations], dtype=np.int64)
    requests = len(reservations)
    padded = pad_to if pad_to is not None else requests
    if pad_tokens_to is None:
        padding = np.ones(padded - requests, np.int64)
    else:
        padding = np.zeros(padded - requests, np.int64)
        missing = pad_tokens_to - int(counts.sum())
        if missing < 0 or (missing > 0 and padded == requests):
            raise ValueError("the step does not fit the shape it is padded to")
        if missing:
            padding[0] = missing
    extra = int(padding.sum())
    all_counts = np.concatenate([counts, padding])
    total = int(all_counts.sum())
    query_start = np.zeros(padded + 1, dtype=np.int32)
    query_start[1:] = np.cumsum(all_counts)
    token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries] + [np.zeros(extra, np.int32)])
    positions = np.concatenate(
        [np.arange(r.start, r.start + r.count, dtype=np.int32) for r in reservations] + [np.zeros(extra, np.int32)]
    )
    token_sequence = np.repeat(np.arange(padded, dtype=np.int32), all_counts)
    context = np.array([r.start + r.count for r in reservations] + [1] * (padded - requests), dtype=np.int32)
    slots = np.array([r.slot for r in reservations] + [cache.spare_slot] * (padded - requests), dtype=np.int32)
    rows = [query_start[b] + np.asarray(e.want, dtype=np.int32) for b, e in enumerate(entries)]
    logit_rows = np.concatenate(rows).astype(np.int32) if rows else np.zeros(0, np.int32)
    wanted = int(logit_rows.size)
    if pad_rows_to is not None:
        logit_rows = np.concatenate([logit_rows, np.zeros(pad_rows_to - wanted, np.int32)])
    elif pad_to is not None:
        logit_rows = np.arange(padded, dtype=np.int32)
    pieces = [token_ids, positions, token_sequence, query_start, context, slots, logit_rows]
    widths = []
    real_slots = slots[:requests]
    for index, group in enumerate(cache.groups):
        needed = max(1, int(-(-int(context.max()) // cache.page_size)))
        group_width = width if width is not None else needed
        widths.append(group_width)
        mapping = np.concatenate([r.slots[index] for r in reservations] + [np.full(extra, -1, np.int32)])
        tables = np.zeros((padded, group_width), dtype=np.int32)
        tables[:requests, : min(needed, group_width)] = group.tables[real_slots, : min(needed, group_width)]
        pieces.append(mapping)
        pieces.append(tables.reshape(-1))
    sizes = [int(piece.size) for piece in pieces]
    facts = {
        "num_tokens": total,
        "num_logit_rows": int(logit_rows.size),
        "wanted": wanted,
        "every_row_wanted": bool(logit_rows.size == total and np.array_equal(logit_rows, np.arange(total, dtype=np.int32))),
        "max_query_length": int(counts.max()),
        "max_context_length": int(context.max()),
        "requests": padded,
    }
    return np.concatenate(pieces).astype(np.int32, copy=False), sizes, widths, facts


def _view_step(
    on_device: torch.Tensor, sizes: list[int], widths: list[int], facts: dict, chunks: list[SequenceChunk], page_size: int,
    padded_to: tuple[int, int] | None = None,
) -> StepBatch:
    views = list(torch.split(on_device, sizes))
    groups = []
    for index, width in enumerate(widths):
        mapping, tables = views[7 + 2 * index], views[8 + 2 * index]
        groups.append(GroupBatch(page_size, tables.view(facts["requests"], width), mapping, width))
    return StepBatch(
        num_tokens=facts["num_tokens"],
        chunks=chunks,
        token_ids=views[0],
        positions=views[1],
        token_sequence=views[2],
        query_start=views[3],
        context_lengths=views[4],
        state_slots=views[5],
        groups=groups,
        logit_rows=views[6],
        num_logit_rows=facts["num_logit_rows"],
        every_row_wanted=facts.get("every_row_wanted", False),
        max_query_length=facts["max_query_length"],
        max_context_length=facts["max_context_length"],
        padded_to=padded_to,
    )


def build_step_batch(
    reservations: list[Reservation],
    entries: list[StepEntry],
    cache: CacheManager,
    device: torch.device,
) -> StepBatch:
    """All index arrays of a step, packed on the host and sent in one copy."""
    packed, sizes, widths, facts = _pack_step(reservations, entries, cache)
    on_device = torch.from_numpy(packed).to(device)
    chunks = [SequenceChunk(r.request_id, r.slot, r.start, r.count) for r in reservations]
    return _view_step(on_device, sizes, widths, facts, chunks, cache.page_size)


@dataclass
class _DecodeGraph:
    """One captured step: `requests` requests (in a decode step one token each) against block tables `width` wide."""

    requests: int
    width: int
    graph: Any
    static: torch.Tensor  # the packed index arrays the captured kernels read
    host: list[torch.Tensor]  # two pinned staging buffers, used in turn
    copied: list[Any]  # per staging buffer: the event after its last copy
    logits: torch.Tensor
    # The captured kernels read the batch's tensors by address, also the work lists that the
    # kernel library keeps on it: the batch lives as long as the graph.
    batch: StepBatch | None = None
    turn: int = 0


class ModelRunner:
    """A model, its cache and the step function over them."""

    def __init__(
        self,
        loaded: LoadedModel,
        kernels,
        cache_config: CacheConfig | None = None,
        *,
        max_sequence_length: int | None = None,
        use_graphs: bool | None = None,
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
        self.use_graphs = self.device.type == "cuda" if use_graphs is None else use_graphs
        self.use_graphs = self.use_graphs and self.model.replayable  # a part that looks at values on the host is not replayed
        self._graphs: dict[tuple[int, int], _DecodeGraph] = {}  # in order of last use, the latest last
        self.max_graphs = 24  # each holds only a step's activations
        # Steps that are not single tokens (prompt portions, portions beside decoded tokens) are captured too,
        # by padded shape, up to this many tokens: below it the host's launches take longer than the device's
        # work.  A shape is captured when it comes for the second time.
        self.graph_token_limit = 512
        self.max_step_graphs = 48
        self._step_graphs: dict[tuple, _DecodeGraph] = {}
        self._shape_seen: dict[tuple, int] = {}
        self._captures_off = False  # set when a capture ran out of memory: graphs that exist are still replayed
        self.step_counts = {"replayed": 0, "captured": 0, "launched": 0}  # how steps reached the device
        self.packing_ms = 0.0  # host time spent on the steps' index arrays
        # What `prepare_decode` has done for the step to come: each request's reservation of one
        # token, and, where decode steps replay a graph, the step's index arrays already packed.
        self._ahead: dict[str, Reservation] = {}
        self._packed_ahead: tuple | None = None

    def close(self) -> None:
        """Drops the captured graphs (while the device runtime is still up)."""
        self._packed_ahead = None
        if self._graphs or self._step_graphs:
            torch.cuda.synchronize(self.device)
        self._graphs.clear()
        self._step_graphs.clear()

    def add_request(self, request_id: str) -> int:
        return self.cache.create(request_id)

    def end_request(self, request_id: str) -> None:
        self._ahead.pop(request_id, None)  # its pages go with the rest
        self.cache.free(request_id)

    def fits(self, plan: list[tuple[str, int]]) -> bool:
        """The cache's `fits` for the step to come; a token that `prepare_decode` has reserved
        already is not counted again."""
        if not self._ahead:
            return self.cache.fits(plan)
        return self.cache.fits([(request_id, count - (1 if request_id in self._ahead else 0)) for request_id, count in plan])

    def prepare_decode(self, request_ids: list[str]) -> bool:
        """Does the host's share of the next step ahead of time, while the device is busy with
        the current one: the step in which each of `request_ids` brings one token and wants its
        logits.  Cache entries are reserved, and the index arrays packed where the step will be
        replayed from a graph; the tokens themselves come with `step`.  A step that turns out
        otherwise costs nothing: reservations of requests it holds are used, the others are
        taken back.  Returns False, having done nothing, if the cache has no room."""
        self._cancel_ahead()
        if not request_ids:
            return False
        plan = [(request_id, 1) for request_id in request_ids]
        if any(request_id not in self.cache.sequences for request_id in request_ids) or not self.cache.fits(plan):
            return False
        reservations = [self.cache.reserve(request_id, 1, checked=True) for request_id in request_ids]
        self._ahead = {r.request_id: r for r in reservations}
        if self.use_graphs:
            entries = [StepEntry(request_id, (0,), (0,)) for request_id in request_ids]
            self._packed_ahead = (tuple(request_ids), *self._pack_decode(reservations, entries))
        return True

    def step_from_device(self, request_ids: list[str], tokens: torch.Tensor) -> torch.Tensor:
        """The step that `prepare_decode(request_ids)` has just prepared, with request i's token taken
        from `tokens[i]`, an integer tensor on the device (the sampler's output for the step before):
        the step is queued behind the work that produces the tokens, and the host never waits for
        them.  Returns what `step` returns."""
        if set(self._ahead) != set(request_ids) or len(tokens) != len(request_ids):
            raise RuntimeError("step_from_device follows prepare_decode for the same requests")
        ahead = self._packed_ahead
        if ahead is None:  # no graphs here (a host run): the tokens are read after all
            entries = [StepEntry(request_id, (int(token),), (0,)) for request_id, token in zip(request_ids, tokens.tolist())]
            return self.step(entries, fits_checked=True)
        reservations = [self._ahead[request_id] for request_id in ahead[0]]
        self._ahead.clear()
        self._packed_ahead = None
        return self._decode_with_graph(reservations, None, ahead[1:], device_tokens=tokens)

    def fetch_later(self, values: torch.Tensor):
        """Queues a copy of a small integer tensor to the host behind the work queued so far; returns a
        function that waits for that copy, and not for what is queued after this call, and gives the
        values as a list."""
        if self.device.type != "cuda":
            return values.tolist
        host = torch.empty(values.shape, dtype=values.dtype, pin_memory=True)
        host.copy_(values, non_blocking=True)
        done = torch.cuda.Event()
        done.record()

        def result() -> list[int]:
            done.synchronize()
            return host.tolist()

        return result

    def _cancel_ahead(self) -> None:
        for reservation in self._ahead.values():
            self.cache.cancel(reservation)
        self._ahead.clear()
        self._packed_ahead = None

    def has_request(self, request_id: str) -> bool:
        return request_id in self.cache.sequences

    def step(self, entries: list[StepEntry], *, create_missing: bool = False, fits_checked: bool = False) -> torch.Tensor:
        """Runs the entries as one batch; returns float32 logits [wanted, vocab]
        in the order of the entries and of each entry's `want`.  The tensor may be a
        view of a buffer that the next step overwrites: use it, or copy it, before then.

        Nothing is reserved if the batch does not fit (`CacheFullError`); `fits_checked`
        says that the caller has asked the cache's `fits` for exactly these entries."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        ahead = self._packed_ahead
        if ahead is not None and len(entries) == len(ahead[0]) and all(
            entry.request_id == request_id and len(entry.tokens) == 1 and tuple(entry.want) == (0,)
            for entry, request_id in zip(entries, ahead[0])
        ):  # the step that `prepare_decode` was told to expect: only the tokens are new
            tokens = [entry.tokens[0] for entry in entries]
            if min(tokens) < 0 or max(tokens) >= self.vocab_size:
                raise ValueError("a token is outside the vocabulary")
            reservations = [self._ahead[request_id] for request_id in ahead[0]]
            self._ahead.clear()
            self._packed_ahead = None
            return self._decode_with_graph(reservations, entries, ahead[1:])
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
            if min(entry.tokens) < 0 or max(entry.tokens) >= self.vocab_size:
                raise ValueError(f"request {entry.request_id!r}: a token is outside the vocabulary")
        created = []
        try:
            for entry in entries:
                if not self.has_request(entry.request_id):
                    if not create_missing:
                        raise KeyError(f"unknown request {entry.request_id!r}")
                    self.add_request(entry.request_id)
                    created.append(entry.request_id)
            plan = [(entry.request_id, len(entry.tokens)) for entry in entries]
            if not fits_checked and not self.fits(plan):
                raise CacheFullError("the step's tokens do not fit the cache")
        except Exception:
            for request_id in created:
                self.end_request(request_id)
            raise
        packed_ahead, self._packed_ahead = self._packed_ahead, None
        reservations = []
        for request_id, count in plan:
            ahead = self._ahead.pop(request_id, None)
            if ahead is not None and count != 1:
                self.cache.cancel(ahead)
                ahead = None
            reservations.append(ahead or self.cache.reserve(request_id, count, checked=True))
        self._cancel_ahead()  # requests that were expected and did not come
        if self.use_graphs and all(len(e.tokens) == 1 and tuple(e.want) == (0,) for e in entries):
            if packed_ahead is not None and packed_ahead[0] == tuple(entry.request_id for entry in entries):
                return self._decode_with_graph(reservations, entries, packed_ahead[1:])
            return self._decode_with_graph(reservations, entries)
        if self.use_graphs:
            logits = self._step_with_graph(reservations, entries)
            if logits is not None:
                return logits
        started = time.perf_counter()
        batch = build_step_batch(reservations, entries, self.cache, self.device)
        self.packing_ms += 1000.0 * (time.perf_counter() - started)
        return self.forward(batch)

    def _stream_scope(self):
        scope = getattr(self.kernels, "stream_scope", None)
        return scope() if scope is not None else contextlib.nullcontext()

    def _replay_scope(self):
        """Tells the kernel library that the step it is about to launch is one a graph will replay (its
        warm-up run and the captured run alike, so that both take the same routes)."""
        scope = getattr(self.kernels, "replay_scope", None)
        return scope() if scope is not None else contextlib.nullcontext()

    @torch.inference_mode()
    def forward(self, batch: StepBatch) -> torch.Tensor:
        with self._stream_scope():
            if batch.num_logit_rows == 0:
                self.model.forward_without_logits(batch, self.cells)
                return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
            return self.model.forward(batch, self.cells)

    # ------------------------------------------------------------------ captured decode steps

    @staticmethod
    def _bucket(value: int) -> int:
        size = 1
        while size < value:
            size *= 2
        return size

    @classmethod
    def _request_bucket(cls, requests: int) -> int:
        """The rows of the graph that a step of so many single tokens replays: a power of two up to 128, where the
        kernels' cost goes by tiles of 16 to 128 rows and padding costs little (65 requests of the 1.5B sizes 2.37 ms a
        step, 128 requests 2.55), and multiples of 64 beyond, where every product is the library's and goes by its rows
        (192 requests take 3.80 ms a step in a graph of 256 rows and 3.66 in one of 192)."""
        return cls._bucket(requests) if requests <= 128 else -(-requests // 64) * 64

    def _pack_decode(self, reservations: list[Reservation], entries: list[StepEntry]):
        """The index arrays of a step of single tokens, padded to its graph's shape; first the graph's key."""
        started = time.perf_counter()
        requests = self._request_bucket(len(reservations))
        blocks = max(-(-(r.start + 1) // self.cache.page_size) for r in reservations)
        width = min(self._bucket(blocks), self._bucket(self.cache.max_blocks_per_sequence))
        packed = _pack_step(reservations, entries, self.cache, pad_to=requests, width=width)
        self.packing_ms += 1000.0 * (time.perf_counter() - started)
        return ((requests, width), *packed)

    @torch.inference_mode()
    def _decode_with_graph(
        self, reservations: list[Reservation], entries: list[StepEntry] | None, packed_ahead=None, device_tokens=None
    ) -> torch.Tensor:
        """A step of single tokens, one per request, replayed from a HIP graph: the launches
        of a decode step cost more on the host than the step takes on the device.  Graphs are
        kept per (requests rounded up to a power of two, block-table width likewise); the
        step's index arrays go into the graph's static buffer and the same kernels run.
        `packed_ahead` is what `_pack_decode` made of the same reservations before the tokens
        were known: the token ids, which lead the arrays, are filled in, from `entries` or, on the
        device, from `device_tokens`."""
        if packed_ahead is not None:
            key, packed, sizes, widths, facts = packed_ahead
            if entries is not None:
                packed[: len(entries)] = [entry.tokens[0] for entry in entries]
        else:
            key, packed, sizes, widths, facts = self._pack_decode(reservations, entries)
        graph = self._graphs.pop(key, None)
        self.step_counts["replayed" if graph is not None else "captured"] += 1
        if graph is None:
            graph = self._capture(key, packed, sizes, widths, facts)
        self._graphs[key] = graph  # the one used last stands last
        turn = graph.turn
        graph.turn = 1 - turn
        if graph.copied[turn] is not None:
            graph.copied[turn].synchronize()  # the staging buffer's last copy has left it
        graph.host[turn].copy_(torch.from_numpy(packed))
        graph.static.copy_(graph.host[turn], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        graph.copied[turn] = event
        if device_tokens is not None:
            graph.static[: len(reservations)].copy_(device_tokens)
        graph.graph.replay()
        return graph.logits[: len(reservations)]

    # ------------------------------------------------------------------ captured steps of any shape

    @staticmethod
    def _token_bucket(tokens: int) -> int:
        for size in (16, 32, 64, 96, 128, 192, 256, 384, 512, 768, 1024):
            if tokens <= size:
                return size
        return -(-tokens // 512) * 512

    @torch.inference_mode()
    def _step_with_graph(self, reservations: list[Reservation], entries: list[StepEntry]) -> torch.Tensor | None:
        """A step of any mix of portions and single tokens, replayed from a HIP graph of its padded shape:
        tokens rounded up to a bucket (the padding belongs to one request more, stored nowhere, read by
        nobody), requests and block-table width to powers of two, the wanted rows to the requests' bucket.
        The kernel library pads its own work lists likewise and makes them anew for every replay
        (`refresh_step`).  Returns None where the step is launched kernel by kernel instead: a kernel library
        without that hook, more tokens than `graph_token_limit`, or a shape that has not come twice yet."""
        if not hasattr(self.kernels, "refresh_step"):
            return None
        tokens = sum(r.count for r in reservations)
        if tokens > self.graph_token_limit:
            self.step_counts["launched"] += 1
            return None
        started = time.perf_counter()
        wanted = sum(len(e.want) for e in entries)
        padded_tokens = self._token_bucket(tokens)
        requests = self._bucket(len(reservations) + 1)  # one more: the request that owns the padding tokens
        blocks = max(-(-(r.start + r.count) // self.cache.page_size) for r in reservations)
        width = min(self._bucket(blocks), self._bucket(self.cache.max_blocks_per_sequence))
        # wanted rows are padded to the requests' bucket (a row a request, as serving wants them) or, where more
        # are wanted, to the tokens' bucket: few shapes
        rows = 0 if wanted == 0 else requests if wanted <= requests else padded_tokens
        key = (padded_tokens, requests, width, rows)
        graph = self._step_graphs.pop(key, None)
        if graph is None:
            seen = self._shape_seen.get(key, 0) + 1
            self._shape_seen[key] = seen
            if seen < 2 or self._captures_off:
                self.step_counts["launched"] += 1
                return None
        self.step_counts["replayed" if graph is not None else "captured"] += 1
        packed, sizes, widths, facts = _pack_step(
            reservations, entries, self.cache, pad_to=requests, width=width, pad_tokens_to=padded_tokens, pad_rows_to=rows
        )
        chunks = [SequenceChunk(r.request_id, r.slot, r.start, r.count) for r in reservations]
        self.packing_ms += 1000.0 * (time.perf_counter() - started)
        if graph is None:
            try:
                graph = self._capture_step(key, packed, sizes, widths, facts, chunks)
            except torch.OutOfMemoryError:
                # no room for another graph's buffers beside the cache: this shape, and new ones from now on,
                # are launched kernel by kernel (the step itself has not run yet: nothing is lost)
                self._captures_off = True
                self.step_counts["captured"] -= 1
                self.step_counts["launched"] += 1
                torch.cuda.empty_cache()
                return None
        self._step_graphs[key] = graph  # the one used last stands last
        turn = graph.turn
        graph.turn = 1 - turn
        if graph.copied[turn] is not None:
            graph.copied[turn].synchronize()  # the staging buffer's last copy has left it
        graph.host[turn].copy_(torch.from_numpy(packed))
        graph.static.copy_(graph.host[turn], non_blocking=True)
        graph.batch.chunks = chunks
        self.kernels.refresh_step(graph.batch, turn)
        event = torch.cuda.Event()
        event.record()
        graph.copied[turn] = event
        graph.graph.replay()
        if wanted == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        return graph.logits[:wanted]

    def _capture_step(self, key, packed, sizes, widths, facts, chunks) -> _DecodeGraph:
        padded_tokens, requests, width, rows = key
        if len(self._step_graphs) >= self.max_step_graphs:
            torch.cuda.synchronize(self.device)  # a replay of the graph that goes may still be queued
            self._step_graphs.pop(next(iter(self._step_graphs)))
        static = torch.from_numpy(packed).to(self.device)
        # what decides which kernels run, and with how many workgroups, is the padded shape and never the step
        facts = dict(facts, max_context_length=width * self.cache.page_size, max_query_length=padded_tokens,
                     every_row_wanted=False)
        batch = _view_step(static, sizes, widths, facts, chunks, self.cache.page_size, padded_to=(padded_tokens, requests))
        stream = torch.cuda.Stream(self.device)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream), self._stream_scope(), self._replay_scope(), self._states_kept():
            self._forward_batch(batch)  # loads libraries, builds the work lists kept on `batch`
        torch.cuda.current_stream(self.device).wait_stream(stream)
        torch.cuda.synchronize(self.device)
        batch.computed.clear()  # what kernels computed from the warm-up's values is recorded anew
        captured = torch.cuda.CUDAGraph()
        with torch.cuda.graph(captured), self._stream_scope(), self._replay_scope():
            logits = self._forward_batch(batch)
        host = [torch.empty(packed.size, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        return _DecodeGraph(requests, width, captured, static, host, [None, None], logits, batch)

    @contextlib.contextmanager
    def _states_kept(self):
        """A step that is being captured runs twice, once launched to warm up and once replayed.  Keys and values
        land in the same places both times; a request's fixed-size state would advance twice, so it is put back
        after the first."""
        saved = [state.clone() for state in self.cache.states]
        try:
            yield
        finally:
            for state, before in zip(self.cache.states, saved):
                state.copy_(before)

    def _forward_batch(self, batch: StepBatch) -> torch.Tensor | None:
        if batch.num_logit_rows == 0:
            self.model.forward_without_logits(batch, self.cells)
            return None
        return self.model.forward(batch, self.cells)

    def _capture(self, key, packed, sizes, widths, facts) -> _DecodeGraph:
        requests, width = key
        if len(self._graphs) >= self.max_graphs:
            # The graph that was used longest ago goes.  A replay of it may still be queued (a step that was
            # queued ahead), and its kernels read the buffers it owns: the device finishes first.
            torch.cuda.synchronize(self.device)
            self._graphs.pop(next(iter(self._graphs)))
        static = torch.from_numpy(packed).to(self.device)
        chunks = [SequenceChunk(f"#{index}", 0, 0, 1) for index in range(requests)]
        # the widest context these tables can describe decides how the attention splits its keys
        facts = dict(facts, max_context_length=width * self.cache.page_size)
        batch = _view_step(static, sizes, widths, facts, chunks, self.cache.page_size)
        stream = torch.cuda.Stream(self.device)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream), self._stream_scope(), self._replay_scope(), self._states_kept():
            self.model.forward(batch, self.cells)  # loads libraries, builds the work lists kept on `batch`
        torch.cuda.current_stream(self.device).wait_stream(stream)
        torch.cuda.synchronize(self.device)
        batch.computed.clear()  # what kernels computed from the warm-up's values is recorded anew
        captured = torch.cuda.CUDAGraph()
        with torch.cuda.graph(captured), self._stream_scope(), self._replay_scope():
            logits = self.model.forward(batch, self.cells)
        host = [torch.empty(packed.size, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        return _DecodeGraph(requests, width, captured, static, host, [None, None], logits, batch)
