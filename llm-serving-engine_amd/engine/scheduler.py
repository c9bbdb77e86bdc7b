"""Iteration-level scheduling: who runs, how many tokens each request brings to a
step, and who gives way when the cache is full.

The behaviour is the reference's (`scheduler.py:40-97` for queues, policies and
admission; `engine.py:255-267,372-400` for the step plan and the choice of a
victim): first-come, shortest-job or priority order, admission every iteration
or only into an empty batch, one token for everybody and then prompt portions
while the step's budget lasts.  The structures are this engine's own: a request
carries its generation settings, the line of waiting requests is a heap keyed
by the policy, and planning and the victim rule are the scheduler's methods,
so every decision the tests check without a model sits in one object.
"""

from __future__ import annotations

import heapq
import time
from collections.abc import Awaitable, Callable
from dataclasses import dataclass, field
from typing import Any, NamedTuple

from ..config.serving import SchedulerConfig
from ..sampling.sampler import GenerationConfig

TokenCallback = Callable[[int], Awaitable[None] | None]


@dataclass(eq=False)
class Request:
    """One request from its arrival to its last token.

    `cached` counts the tokens of prompt + output whose keys and values the
    cache holds; what is still `owed` to the model is the rest.  A request that
    gave way starts again at `cached = 0` and replays prompt and output without
    emitting anything until it has caught up.
    """

    request_id: str
    prompt: list[int]
    settings: GenerationConfig = field(default_factory=GenerationConfig)
    priority: int = 0
    on_token: TokenCallback | None = None
    output: list[int] = field(default_factory=list)
    cached: int = 0
    ticket: int = -1  # arrival number, given by the scheduler; ties in every policy go to the lower
    arrived_at: float = field(default_factory=time.monotonic)
    admitted_at: float | None = None  # first admission
    evictions: int = 0  # times it gave way
    replayed_tokens: int = 0  # tokens computed again because of that
    outcome: Any = None  # a future, for the asynchronous entry point
    error: Exception | None = None
    done: bool = False

    @property
    def length(self) -> int:
        return len(self.prompt) + len(self.output)

    @property
    def owed(self) -> int:
        return self.length - self.cached

    @property
    def output_left(self) -> int:
        return self.settings.max_new_tokens - len(self.output)

    @property
    def in_prompt(self) -> bool:
        return self.cached < len(self.prompt)

    def next_tokens(self, count: int) -> list[int]:
        """The `count` tokens after the cached ones (a decode step asks for one: no list is joined for it)."""
        first, last, border = self.cached, self.cached + count, len(self.prompt)
        if first >= border:
            return self.output[first - border : last - border]
        if last <= border:
            return self.prompt[first:last]
        return self.prompt[first:] + self.output[: last - border]


class Share(NamedTuple):
    """A request's share of one step."""

    request: Request
    count: int


_ORDERINGS: dict[str, Callable[[Request], tuple]] = {
    "fcfs": lambda request: (request.ticket,),
    "sjf": lambda request: (request.output_left, request.ticket),
    "priority": lambda request: (-request.priority, request.ticket),
}


class Scheduler:
    """The line of waiting requests and the running batch.

    A request's place in the line is fixed when it joins it (its key cannot
    change while it waits: output is produced only while running), so the line
    is a heap and admission pops its head.  A request that gives way rejoins
    with its old ticket: under first-come order it is the next to be admitted.
    """

    def __init__(self, limits: SchedulerConfig | None = None, mode: str = "continuous") -> None:
        self.limits = limits or SchedulerConfig()
        if self.limits.policy not in _ORDERINGS:
            raise ValueError(f"policy must be one of {', '.join(_ORDERINGS)}")
        if mode not in ("continuous", "static"):
            raise ValueError("mode must be continuous or static")
        if self.limits.max_batch_size <= 0:
            raise ValueError("max_batch_size must be positive")
        if self.limits.preemption not in ("largest", "latest"):
            raise ValueError("preemption must be largest or latest")
        self.mode = mode
        self.running: list[Request] = []
        self._line: list[tuple[tuple, Request]] = []
        self._key = _ORDERINGS[self.limits.policy]
        self._tickets = 0

    # ------------------------------------------------------------------ the line

    def enqueue(self, request: Request) -> None:
        request.ticket = self._tickets
        self._tickets += 1
        heapq.heappush(self._line, (self._key(request), request))

    @property
    def waiting(self) -> list[Request]:
        """The line in the order in which it would be admitted."""
        return [request for _, request in sorted(self._line, key=lambda item: item[0])]

    @property
    def num_waiting(self) -> int:
        return len(self._line)

    @property
    def idle(self) -> bool:
        return not self._line and not self.running

    def admit(self) -> list[Request]:
        """Moves requests from the head of the line into the batch: every iteration while
        there is room (continuous), or only into an empty batch (static).  Memory is not
        asked about here (`scheduler.py:75-83`): pages are found, or somebody gives way,
        when the step is planned."""
        if self.mode == "static" and self.running:
            return []
        admitted = []
        now = time.monotonic()
        while self._line and len(self.running) < self.limits.max_batch_size:
            _, request = heapq.heappop(self._line)
            if request.admitted_at is None:
                request.admitted_at = now
            self.running.append(request)
            admitted.append(request)
        return admitted

    def retire(self, request: Request) -> None:
        """Takes the request out of the batch, or out of the line."""
        if request in self.running:
            self.running.remove(request)
        else:
            remaining = [item for item in self._line if item[1] is not request]
            if len(remaining) != len(self._line):
                self._line = remaining
                heapq.heapify(self._line)

    def evict(self, request: Request) -> None:
        """The request gives way: back into the line, everything it had cached to be
        computed again (`scheduler.py:88-93`)."""
        self.running.remove(request)
        request.replayed_tokens += request.cached
        request.cached = 0
        request.evictions += 1
        heapq.heappush(self._line, (self._key(request), request))

    # ------------------------------------------------------------------ one step

    def plan(self, chunk: int) -> list[Share]:
        """Everybody in the batch brings one token; what the step's budget then has left
        goes, in batch order, to requests that owe more, up to `chunk` tokens each
        (`engine.py:372-391`).  A decoding request owes one token and stays at one."""
        spare = self.limits.max_tokens_per_step - len(self.running)
        shares = []
        for request in self.running:
            if request.owed <= 0:
                raise RuntimeError(f"request {request.request_id!r} is in the batch and owes no token")
            more = min(max(spare, 0), min(chunk, request.owed) - 1)
            spare -= more
            shares.append(Share(request, 1 + more))
        return shares

    def victim(self, shares: list[Share]) -> Request:
        """Who gives way when the step's pages do not fit.

        "largest": the one with most tokens cached (`engine.py:258`): it frees most
        pages, at the price of most recomputation.  "latest": the one that arrived
        last.  Under both, the request that arrived first never gives way.  The
        reference has no such exemption, and with its rule two requests that cannot
        both fit may evict each other for ever, each overtaking the other while it
        replays; with the exemption the oldest always finishes, then the next oldest.
        """
        requests = [share.request for share in shares]
        eldest = min(requests, key=lambda request: request.ticket)
        others = [request for request in requests if request is not eldest]
        if not others:
            raise ValueError("a single request cannot give way to itself")
        if self.limits.preemption == "largest":
            return max(others, key=lambda request: (request.cached, -request.ticket))
        return max(others, key=lambda request: request.ticket)
