"""The cache manager: pages with a block table per request, one pool per group of
layers with the same need, and slots of fixed-size state.

The reference keeps one tensor [L, 2, NB, P, Hkv, D] for all layers, one block
table per sequence and a metadata row per sequence (`kv_cache.py:91-179`).  Here
the layers that run are first sorted into groups by what their parts need: an
entry per token (`PagedNeed`: all of them, or a window) or an entry per request
(`SlotNeed`); a run may need several things at once.  Every paged group has its
own pool, block tables and, for each field its need names, a tensor [cells, NB,
*page shape]: what a page holds is the need's business (keys and values for
attention), the manager only hands pages out and takes them back, and a windowed
group gives a page back as soon as no later query can read it.  A request's slot
(the reference's metadata row) is its block-table row in every group and its
index into every per-request tensor.
"""

from __future__ import annotations

import math
from collections import deque
from dataclasses import dataclass, field

import numpy as np
import torch

from ..config.serving import CacheConfig
from .cell import CacheCell
from ..parts.base import CacheNeed, PagedNeed, SlotNeed
from ..parts.model import ModelSpec
from .pool import CacheFullError, PagePool


@dataclass
class PageGroup:
    need: PagedNeed
    cells: list[tuple[int, str | None]]  # (run of the run order, name of the need in that run) of every cell here
    pool: PagePool
    storage: dict[str, torch.Tensor]  # by field of the need: [len(cells), NB, *page shape]
    tables: np.ndarray  # int32 [max_sequences, max_blocks]; -1 where no page is held
    peak_pages: int = 0

    @property
    def bytes_per_page(self) -> int:
        """What one page takes over all cells and fields of the group."""
        return sum(tensor[:, 0].numel() * tensor.element_size() for tensor in self.storage.values())


@dataclass
class SequenceRecord:
    request_id: str
    slot: int
    length: int = 0
    # per group: number of leading logical blocks already given back (window passed)
    released: list[int] = field(default_factory=list)
    last_access_tick: int = 0


@dataclass(frozen=True)
class Reservation:
    """Where the next `count` tokens of a request go."""

    request_id: str
    slot: int
    start: int
    count: int
    slots: tuple[np.ndarray, ...]  # per group: int32 [count], page * page_size + offset


class CacheManager:
    def __init__(
        self,
        spec: ModelSpec,
        config: CacheConfig,
        *,
        max_sequence_length: int,
        dtype: torch.dtype = torch.float32,
        device: str | torch.device = "cpu",
    ) -> None:
        self.spec = spec
        self.config = config
        self.dtype = dtype
        self.device = torch.device(device)
        self.page_size = config.block_size
        self.max_sequence_length = max_sequence_length
        self.max_blocks_per_sequence = math.ceil(max_sequence_length / config.block_size)
        self.sequences: dict[str, SequenceRecord] = {}
        self._free_slots: deque[int] = deque(range(config.max_sequences))
        self._tick = 0
        self._used_tokens = 0  # tokens cached over all live requests
        self._high_water = {"pages": 0, "used_tokens": 0, "sequences": 0}

        self.groups: list[PageGroup] = []
        # per run: by name of the need (None for a run with one need) -> (kind, group or state index, index inside)
        self._cell_of_run: list[dict[str | None, tuple[str, int, int]]] = []
        self.states: list[torch.Tensor] = []
        self._state_needs: list[SlotNeed] = []
        by_need: dict[PagedNeed, int] = {}
        for index, run in enumerate(spec.run_order):
            if run.reads is not None:
                self._cell_of_run.append(self._cell_of_run[run.reads])
                continue
            entries: dict[str | None, tuple[str, int, int]] = {}
            for name, need in self._named(spec.cell_need(index), index).items():
                if isinstance(need, PagedNeed):
                    if need not in by_need:
                        by_need[need] = len(self.groups)
                        tables = np.full((config.max_sequences, self.max_blocks_per_sequence), -1, np.int32)
                        self.groups.append(PageGroup(need, [], PagePool(config.num_blocks), {}, tables))
                    group = by_need[need]
                    self.groups[group].cells.append((index, name))
                    entries[name] = ("pages", group, len(self.groups[group].cells) - 1)
                elif isinstance(need, SlotNeed):
                    self._state_needs.append(need)
                    # one slot more than there are requests: the state of the requests that pad a captured step
                    self.states.append(
                        torch.zeros((config.max_sequences + 1, *need.shape), dtype=torch.float32, device=self.device)
                    )
                    entries[name] = ("state", len(self.states) - 1, 0)
                else:
                    raise TypeError(f"run {index}: a cache need is a PagedNeed or a SlotNeed, not {need!r}")
            self._cell_of_run.append(entries)
        for group in self.groups:
            for field_name, shape in group.need.page_fields(self.page_size).items():
                group.storage[field_name] = torch.zeros(
                    (len(group.cells), config.num_blocks, *shape), dtype=dtype, device=self.device
                )

    @staticmethod
    def _named(need: "CacheNeed | dict[str, CacheNeed] | None", run: int) -> dict[str | None, CacheNeed]:
        """A run's needs by name: none, one (under None), or the several its block named."""
        if need is None:
            return {}
        if isinstance(need, dict):
            if any(not isinstance(name, str) for name in need):
                raise TypeError(f"run {run}: several cache needs are named by strings")
            return {name: value for name, value in need.items() if value is not None}
        return {None: need}

    # ------------------------------------------------------------------ views

    def _cell(self, entry: tuple[str, int, int], writable: bool) -> CacheCell:
        if entry[0] == "pages":
            group = self.groups[entry[1]]
            fields = {name: tensor[entry[2]] for name, tensor in group.storage.items()}
            return CacheCell(need=group.need, writable=writable, group=entry[1], fields=fields)
        return CacheCell(need=self._state_needs[entry[1]], writable=writable, state=self.states[entry[1]])

    def cells(self) -> list["CacheCell | dict[str, CacheCell] | None"]:
        """One entry per entry of the run order, in order: the run's cell, None for a run that keeps
        nothing, or the cells by name for a run whose block named several needs."""
        views: list[CacheCell | dict[str, CacheCell] | None] = []
        for index, entries in enumerate(self._cell_of_run):
            writable = self.spec.run_order[index].reads is None
            if not entries:
                views.append(None)
            elif None in entries:
                views.append(self._cell(entries[None], writable))
            else:
                views.append({name: self._cell(entry, writable) for name, entry in entries.items()})
        return views

    # ------------------------------------------------------------------ requests

    def create(self, request_id: str) -> int:
        """Gives the request a slot: an empty block-table row in every group and
        zeroed fixed state (reference `kv_cache.py:135-143`)."""
        if request_id in self.sequences:
            raise ValueError(f"sequence {request_id!r} already exists")
        if not self._free_slots:
            raise CacheFullError("paged cache has no free request slots")
        slot = self._free_slots.popleft()
        for group in self.groups:
            group.tables[slot].fill(-1)
        for state in self.states:
            state[slot].zero_()
        self.sequences[request_id] = SequenceRecord(request_id, slot, released=[0] * len(self.groups))
        return slot

    def _first_needed_block(self, group: PageGroup, start: int) -> int:
        """Blocks below this index hold no key that a query at position >= start reads."""
        if group.need.window is None:
            return 0
        return max(0, start - group.need.window + 1) // self.page_size

    def pages_needed(self, request_id: str, count: int) -> list[tuple[int, int]]:
        """Per group: (pages to allocate, pages given back first) for the next `count` tokens."""
        record = self.sequences[request_id]
        need = []
        for index, group in enumerate(self.groups):
            held_until = math.ceil(record.length / self.page_size)
            wanted_until = math.ceil((record.length + count) / self.page_size)
            first = self._first_needed_block(group, record.length)
            giving_back = max(0, min(first, held_until) - record.released[index])
            need.append((wanted_until - held_until, giving_back))
        return need

    def fits(self, plan: list[tuple[str, int]]) -> bool:
        """Whether every (request, count) of `plan` can be reserved, in order."""
        free = [group.pool.free_pages for group in self.groups]
        for request_id, count in plan:
            record = self.sequences[request_id]
            if record.length + count > self.max_sequence_length:
                return False
            for index, (allocate, give_back) in enumerate(self.pages_needed(request_id, count)):
                free[index] += give_back - allocate
                if free[index] < 0:
                    return False
        return True

    def pages_short(self, plan: list[tuple[str, int]]) -> int:
        """How many pages are missing, summed over groups, to reserve all of `plan`."""
        short = 0
        for index, group in enumerate(self.groups):
            balance = group.pool.free_pages
            for request_id, count in plan:
                allocate, give_back = self.pages_needed(request_id, count)[index]
                balance += give_back - allocate
            short += max(0, -balance)
        return short

    def reserve(self, request_id: str, count: int, *, checked: bool = False) -> Reservation:
        """Takes the cache entries of the request's next `count` tokens
        (reference `kv_cache.py:145-179`).  Pages that a window has passed are
        given back first.  Raises `CacheFullError`, holding nothing new, if a
        pool runs dry or the request would outgrow the longest sequence;
        `checked` says that the caller has asked `fits` for this already."""
        if count <= 0:
            raise ValueError("count must be positive")
        record = self.sequences[request_id]
        start = record.length
        if not checked:
            if start + count > self.max_sequence_length:
                raise CacheFullError("sequence exceeds the longest sequence the cache was built for")
            if not self.fits([(request_id, count)]):
                raise CacheFullError("paged cache has no free pages")
        page_size = self.page_size
        first_new = -(-start // page_size)
        end_new = -(-(start + count) // page_size)
        slots = []
        for index, group in enumerate(self.groups):
            table = group.tables[record.slot]
            if group.need.window is not None:
                first = min(self._first_needed_block(group, start), first_new)
                for block in range(record.released[index], first):
                    group.pool.free(int(table[block]), request_id)
                    table[block] = -1
                if first > record.released[index]:
                    record.released[index] = first
            for block in range(first_new, end_new):
                table[block] = group.pool.allocate(request_id)
            if group.pool.used_pages > group.peak_pages:
                group.peak_pages = group.pool.used_pages
            if count == 1:  # a decoded token: no arrays on the way
                slots.append(np.array([int(table[start // page_size]) * page_size + start % page_size], np.int32))
            else:
                positions = np.arange(start, start + count)
                pages = table[positions // page_size].astype(np.int64)
                slots.append((pages * page_size + positions % page_size).astype(np.int32))
        record.length = start + count
        self._used_tokens += count
        self._touch(record)
        used = self.used_pages
        if used >= self._high_water["pages"]:
            self._high_water = {"pages": used, "used_tokens": self._used_tokens, "sequences": len(self.sequences)}
        return Reservation(request_id, record.slot, start, count, tuple(slots))

    def cancel(self, reservation: Reservation) -> None:
        """Takes back the request's latest reservation, whose entries were never written: the
        request is as long as before, and pages that the reservation began are free again.
        (Pages that a window had passed stay given back: no later query reads them.)"""
        record = self.sequences[reservation.request_id]
        if record.length != reservation.start + reservation.count:
            raise ValueError(f"not the latest reservation of {reservation.request_id!r}")
        first_new = -(-reservation.start // self.page_size)
        end_new = -(-record.length // self.page_size)
        for group in self.groups:
            table = group.tables[record.slot]
            for block in range(first_new, end_new):
                group.pool.free(int(table[block]), reservation.request_id)
                table[block] = -1
        record.length = reservation.start
        self._used_tokens -= reservation.count

    def block_table(self, request_id: str, group: int = 0) -> list[int]:
        record = self.sequences[request_id]
        blocks = math.ceil(record.length / self.page_size)
        return self.groups[group].tables[record.slot, :blocks].tolist()

    # ------------------------------------------------------------------ host-side read paths

    def _paged_cell(self, run: int, name: str | None = None) -> tuple[PageGroup, int, int]:
        entries = self._cell_of_run[run] if 0 <= run < len(self._cell_of_run) else {}
        entry = entries.get(name)
        if entry is None or entry[0] != "pages":
            raise ValueError(f"run {run} of the run order keeps no pages" + (f" under {name!r}" if name else ""))
        return self.groups[entry[1]], entry[1], entry[2]

    def iter_page_fields(self, request_id: str, run: int, name: str | None = None):
        """Walks what run `run` of the run order has cached for the request (under `name`, for a run with
        several needs), page by page in logical order: yields (first position, {field: [n, ...]}), the
        token's place in the page leading (the need's `token_rows`), the last page cut at the request's
        length, pages that a window has given back left out.  A debugging and testing aid, as the
        reference's `iter_kv_blocks` (`kv_cache.py:268-296`): the kernels read through the block tables
        themselves."""
        group, group_index, cell = self._paged_cell(run, name)
        record = self.sequences[request_id]
        table = group.tables[record.slot]
        page_size = self.page_size
        for block in range(record.released[group_index], math.ceil(record.length / page_size)):
            held = min(page_size, record.length - block * page_size)
            page = {field: tensor[cell, int(table[block])] for field, tensor in group.storage.items()}
            rows = group.need.token_rows(page, page_size)
            yield block * page_size, {field: tensor[:held] for field, tensor in rows.items()}

    def iter_pages(self, request_id: str, run: int, name: str | None = None):
        """`iter_page_fields` for keys and values: yields (first position, keys [n, kv_heads, head_dim],
        values [n, kv_heads, head_dim])."""
        for first, rows in self.iter_page_fields(request_id, run, name):
            yield first, rows["keys"], rows["values"]

    def gather_fields(self, request_id: str, run: int, name: str | None = None) -> tuple[int, dict[str, torch.Tensor]]:
        """(first cached position, {field: [n, ...]}) of the request in run `run`, each field one contiguous tensor."""
        pages = list(self.iter_page_fields(request_id, run, name))
        if not pages:
            return self.sequences[request_id].length, {}
        return pages[0][0], {field: torch.cat([rows[field] for _, rows in pages]) for field in pages[0][1]}

    def gather(self, request_id: str, run: int, name: str | None = None) -> tuple[int, torch.Tensor, torch.Tensor]:
        """(first cached position, keys, values) of the request in run `run` as two contiguous tensors
        [n, kv_heads, head_dim] (`kv_cache.py:318-342`)."""
        first, fields = self.gather_fields(request_id, run, name)
        if not fields:
            need = self._paged_cell(run, name)[0].need
            empty = torch.empty((0, need.num_kv_heads, need.head_dim), dtype=self.dtype, device=self.device)
            return first, empty, empty.clone()
        return first, fields["keys"], fields["values"]

    def block_table_tensors(self, request_ids: list[str], group: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
        """A compact [requests, widest] block table (-1 where nothing is held) and the requests'
        lengths, both int32 on the host (`kv_cache.py:298-316`)."""
        records = [self.sequences[request_id] for request_id in request_ids]
        widest = max((math.ceil(record.length / self.page_size) for record in records), default=0)
        tables = np.stack([self.groups[group].tables[record.slot, :widest] for record in records]) if records else np.zeros((0, 0), np.int32)
        lengths = np.array([record.length for record in records], dtype=np.int32)
        return torch.from_numpy(tables.copy()), torch.from_numpy(lengths)

    def free(self, request_id: str) -> None:
        """Gives back everything the request holds (reference `kv_cache.py:344-350`)."""
        record = self.sequences.pop(request_id)
        self._used_tokens -= record.length
        for group in self.groups:
            table = group.tables[record.slot]
            for page in table[table >= 0].tolist():
                group.pool.free(page, request_id)
            table.fill(-1)
        self._free_slots.append(record.slot)

    def evict(self, policy: str = "largest", exclude: set[str] | None = None) -> tuple[str, int]:
        """Frees one request chosen by `policy` and returns (its id, tokens to
        recompute) (reference `kv_cache.py:352-369`)."""
        candidates = [
            record for record in self.sequences.values() if not exclude or record.request_id not in exclude
        ]
        if not candidates:
            raise CacheFullError("no evictable sequences")
        if policy == "largest":
            victim = max(candidates, key=lambda item: (item.length, -item.last_access_tick))
        elif policy == "lru":
            victim = min(candidates, key=lambda item: item.last_access_tick)
        else:
            raise ValueError(f"unknown eviction policy: {policy}")
        recompute = victim.length
        self.free(victim.request_id)
        return victim.request_id, recompute

    def _touch(self, record: SequenceRecord) -> None:
        self._tick += 1
        record.last_access_tick = self._tick

    # ------------------------------------------------------------------ accounting

    @property
    def free_pages(self) -> int:
        """Free pages of the fullest group."""
        return min((group.pool.free_pages for group in self.groups), default=0)

    @property
    def used_pages(self) -> int:
        return sum(group.pool.used_pages for group in self.groups)

    @property
    def capacity_tokens(self) -> int:
        return self.config.num_blocks * self.page_size

    @property
    def spare_slot(self) -> int:
        """The state slot of requests that only pad a step to a captured shape: real requests never get it."""
        return self.config.max_sequences

    @property
    def bytes_per_token(self) -> int:
        """What one cached token takes over all runs of the run order that keep pages."""
        return sum(group.bytes_per_page for group in self.groups) // self.page_size

    def check_invariants(self) -> None:
        """No page lost, held twice, or held by a request that is gone."""
        for index, group in enumerate(self.groups):
            held: dict[int, str] = {}
            for record in self.sequences.values():
                table = group.tables[record.slot]
                blocks = math.ceil(record.length / self.page_size)
                for block in range(self.max_blocks_per_sequence):
                    page = int(table[block])
                    live = record.released[index] <= block < blocks
                    if live != (page >= 0):
                        raise AssertionError(f"group {index}: {record.request_id} block {block} holds {page}")
                    if page >= 0:
                        if page in held:
                            raise AssertionError(f"group {index}: page {page} held twice")
                        held[page] = record.request_id
            for page, owner in held.items():
                if group.pool.owner_of(page) != owner:
                    raise AssertionError(f"group {index}: page {page} owner mismatch")
            if group.pool.used_pages != len(held):
                raise AssertionError(f"group {index}: {group.pool.used_pages} pages out, {len(held)} in tables")
            if group.pool.used_pages + group.pool.free_pages != group.pool.num_pages:
                raise AssertionError(f"group {index}: pages lost")
            live_slots = {record.slot for record in self.sequences.values()}
            for slot in range(self.config.max_sequences):
                if slot not in live_slots and (group.tables[slot] >= 0).any():
                    raise AssertionError(f"group {index}: free slot {slot} still holds pages")
        if len(self._free_slots) + len(self.sequences) != self.config.max_sequences:
            raise AssertionError("request slots lost")
        if self._used_tokens != sum(record.length for record in self.sequences.values()):
            raise AssertionError("token count drifted")

    def stats(self, contiguous_max_length: int | None = None) -> dict[str, float]:
        """The reference's accounting (`kv_cache.py:386-413`), summed over groups."""
        used_tokens = self._used_tokens
        used = self.used_pages
        total = sum(group.pool.num_pages for group in self.groups)
        held_tokens = 0
        for index, group in enumerate(self.groups):
            for record in self.sequences.values():
                held_tokens += record.length - record.released[index] * self.page_size
        allocated_slots = used * self.page_size
        waste = allocated_slots - held_tokens
        allocated_bytes = sum(group.pool.used_pages * group.bytes_per_page for group in self.groups)
        peak_bytes = sum(group.peak_pages * group.bytes_per_page for group in self.groups)
        result = {
            "blocks_used": float(used),
            "blocks_free": float(total - used),
            "used_tokens": float(used_tokens),
            "paged_waste_tokens": float(waste),
            "paged_fragmentation_pct": 100.0 * waste / max(allocated_slots, 1),
            "paged_allocated_gb": allocated_bytes / 1024**3,
            "peak_blocks_used": float(self._high_water["pages"]),
            "peak_paged_allocated_gb": peak_bytes / 1024**3,
        }
        if contiguous_max_length is not None:
            bytes_per_token = sum(group.bytes_per_page for group in self.groups) / self.page_size
            contiguous_slots = self._high_water["sequences"] * contiguous_max_length
            contiguous_waste = max(contiguous_slots - self._high_water["used_tokens"], 0)
            paged_slots = self._high_water["pages"] * self.page_size / max(len(self.groups), 1)
            result.update(
                contiguous_waste_tokens=float(contiguous_waste),
                contiguous_waste_gb=contiguous_waste * bytes_per_token / 1024**3,
                memory_reduction_pct=100.0 * (contiguous_slots - paged_slots) / max(contiguous_slots, 1),
            )
        return result
