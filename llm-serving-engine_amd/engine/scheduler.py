"""Iteration-level scheduling: who is admitted, how many tokens each request
brings to a step, and who gives way when the cache is full.

Queues, policies and admission follow the reference's `IterationScheduler`
(`scheduler.py:40-97`); the step plan and the victim choice follow its engine
(`engine.py:255-267,372-400`).  They sit together here because both are
decisions, made on the host, that the tests check without a model.
"""

from __future__ import annotations

import itertools
import time
from collections.abc import Awaitable, Callable
from dataclasses import dataclass, field
from typing import Any

TokenCallback = Callable[[int], Awaitable[None] | None]


@dataclass
class RequestState:
    """`scheduler.py:12-37`."""

    request_id: str
    prompt_token_ids: list[int]
    max_new_tokens: int
    callback: TokenCallback | None = None
    priority: int = 0
    arrival_order: int = 0
    arrival_time: float = field(default_factory=time.monotonic)
    generated_token_ids: list[int] = field(default_factory=list)
    processed_tokens: int = 0
    preemptions: int = 0
    recomputed_tokens: int = 0
    future: Any = None
    error: Exception | None = None
    finished: bool = False

    @property
    def all_tokens(self) -> list[int]:
        return self.prompt_token_ids + self.generated_token_ids

    def tokens_between(self, start: int, end: int) -> list[int]:
        """all_tokens[start:end] without joining the two lists (a decode step asks for one token)."""
        prompt = len(self.prompt_token_ids)
        if start >= prompt:
            return self.generated_token_ids[start - prompt : end - prompt]
        if end <= prompt:
            return self.prompt_token_ids[start:end]
        return self.prompt_token_ids[start:] + self.generated_token_ids[: end - prompt]

    @property
    def remaining_input_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.generated_token_ids) - self.processed_tokens

    @property
    def remaining_output_tokens(self) -> int:
        return self.max_new_tokens - len(self.generated_token_ids)

    @property
    def in_prefill(self) -> bool:
        return self.processed_tokens < len(self.prompt_token_ids)


class IterationScheduler:
    """Waiting and active lists with first-come, shortest-job or priority order,
    admitting every iteration (continuous) or only into an empty batch (static)."""

    def __init__(self, max_batch_size: int, policy: str = "fcfs", mode: str = "continuous") -> None:
        if policy not in {"fcfs", "sjf", "priority"}:
            raise ValueError("policy must be fcfs, sjf, or priority")
        if mode not in {"continuous", "static"}:
            raise ValueError("mode must be continuous or static")
        if max_batch_size <= 0:
            raise ValueError("max_batch_size must be positive")
        self.max_batch_size = max_batch_size
        self.policy = policy
        self.mode = mode
        self.waiting: list[RequestState] = []
        self.active: list[RequestState] = []
        self._counter = itertools.count()

    def add(self, request: RequestState) -> None:
        request.arrival_order = next(self._counter)
        self.waiting.append(request)

    def _order(self, request: RequestState):
        if self.policy == "fcfs":
            return (request.arrival_order,)
        if self.policy == "sjf":
            return (request.remaining_output_tokens, request.arrival_order)
        return (-request.priority, request.arrival_order)

    def admit(self) -> list[RequestState]:
        """`scheduler.py:75-83`: no memory check here; pages are found, or a
        request gives way, when the step is planned."""
        if self.mode == "static" and self.active:
            return []
        self.waiting.sort(key=self._order)
        count = min(self.max_batch_size - len(self.active), len(self.waiting))
        admitted = self.waiting[:count]
        del self.waiting[:count]
        self.active.extend(admitted)
        return admitted

    def finish(self, request: RequestState) -> None:
        self.active.remove(request)

    def preempt(self, request: RequestState) -> None:
        """`scheduler.py:88-93`: back to the waiting list with its arrival order
        kept; everything it had processed will be computed again."""
        self.active.remove(request)
        request.recomputed_tokens += request.processed_tokens
        request.processed_tokens = 0
        request.preemptions += 1
        self.waiting.append(request)

    @property
    def empty(self) -> bool:
        return not self.waiting and not self.active


def plan_iteration(
    active: list[RequestState], max_tokens_per_step: int, prefill_chunk_size: int
) -> list[tuple[RequestState, int]]:
    """Every active request gets one token; what is left of the step's budget
    then tops requests up, in order, to `prefill_chunk_size` tokens or to what
    they still have to process (`engine.py:372-391`).  A decoding request has one
    token left and stays at one."""
    budget = max_tokens_per_step
    planned: list[tuple[RequestState, int]] = []
    for request in active:
        if request.remaining_input_tokens <= 0:
            raise RuntimeError("active request has no input token to process")
        planned.append((request, 1))
        budget -= 1
    for index, (request, count) in enumerate(planned):
        if budget <= 0:
            break
        desired = min(prefill_chunk_size, request.remaining_input_tokens)
        extra = min(desired - count, budget)
        planned[index] = (request, count + extra)
        budget -= extra
    return planned


def choose_victim(planned: list[tuple[RequestState, int]], policy: str = "largest") -> RequestState:
    """Who gives way when the step's pages do not fit.

    "largest": the planned request that has processed most tokens
    (`engine.py:258`): it frees most pages, at the price of most recomputation.
    "latest": the one that arrived last.  Under both the request that arrived
    first never gives way.  The reference has no such exemption, and with its
    rule two requests that cannot both fit may evict each other for ever, each
    overtaking the other while it replays; with the exemption the oldest
    request always finishes, then the next oldest.
    """
    if policy not in ("largest", "latest"):
        raise ValueError("preemption must be largest or latest")
    oldest = min(planned, key=lambda item: item[0].arrival_order)[0]
    candidates = [item[0] for item in planned if item[0] is not oldest]
    if not candidates:
        raise ValueError("a single request cannot give way to itself")
    if policy == "largest":
        return max(candidates, key=lambda request: request.processed_tokens)
    return max(candidates, key=lambda request: request.arrival_order)
