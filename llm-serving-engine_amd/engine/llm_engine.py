"""The engine above the step function: it admits requests, plans each
iteration, makes room when pages run out, samples, streams and finishes.

`EngineCore` is the synchronous loop body (one call of `step()` is one
iteration).  `LLMEngine` is the asynchronous entry point with the reference's
interface (`engine.py:108-464`): `await engine.generate(prompt, config,
callback, priority=, request_id=)`.
"""

from __future__ import annotations

import asyncio
import collections
import inspect
import time
import uuid
from dataclasses import dataclass
from typing import Any

import torch

from ..cache.pool import CacheFullError
from ..config.serving import CacheConfig, SchedulerConfig
from ..sampling.sampler import GenerationConfig, Sampler
from ..weights.loader import LoadedModel, load_model_folder
from .runner import ModelRunner, StepEntry
from .scheduler import Request, Scheduler, Share, TokenCallback
from .tokenizer import ByteTokenizer, Tokenizer


class RequestTooLongError(ValueError):
    """Prompt plus the tokens asked for exceed the longest sequence the cache can describe."""


@dataclass
class TokenEvent:
    request: Request
    token: int


@dataclass
class _StepInFlight:
    """A decode step that was queued before the tokens it consumes had reached the host."""

    requests: list[Request]  # row i of `logits` is requests[i]
    logits: torch.Tensor


_PHASES = ("prefill", "decode", "mixed")


class EngineCore:
    """One iteration at a time over a `ModelRunner`."""

    def __init__(
        self,
        runner: ModelRunner,
        scheduler_config: SchedulerConfig | None = None,
        *,
        scheduler_mode: str = "continuous",
        prefill_chunk_size: int = 16,
        collect_iteration_metrics: bool = False,
        look_ahead: bool = True,
        run_ahead: bool = True,
    ) -> None:
        limits = scheduler_config or SchedulerConfig()
        if prefill_chunk_size <= 0:
            raise ValueError("prefill_chunk_size must be positive")
        if limits.max_tokens_per_step < limits.max_batch_size:
            raise ValueError("max_tokens_per_step must allow one token per active request")
        if limits.max_batch_size > runner.cache_config.max_sequences:
            raise ValueError("max_batch_size exceeds the cache's request slots (CacheConfig.max_sequences)")
        self.runner = runner
        self.scheduler_config = limits
        self.scheduler = Scheduler(limits, scheduler_mode)
        self.prefill_chunk_size = prefill_chunk_size
        self.sampler = Sampler(runner.kernels)
        self.collect_iteration_metrics = collect_iteration_metrics
        self.look_ahead = look_ahead  # prepare the next decode step on the host while the device runs this one
        self._expected: list[Request] | None = None  # the requests of the step that is prepared
        # Queue the next decode step behind the sampling of this one, its tokens passed on the device:
        # the device then never waits for the host between two steps.  A request that turns out to have
        # ended (a stop token) has a row in that step that nobody reads.
        self.run_ahead = run_ahead and look_ahead
        self._in_flight: _StepInFlight | None = None
        self._known: set[str] = set()  # ids of requests that are waiting or running
        self.finished: list[Request] = []
        self._host_ms = dict.fromkeys(_PHASES, 0.0)
        self._iterations = dict.fromkeys(_PHASES, 0)
        self._device_spans: dict[str, list] = {phase: [] for phase in _PHASES}
        self._evictions_of_finished = 0
        self._replayed_by_finished = 0
        self.step_log: list[list[tuple[str, int]]] | None = None  # tests set it to [] to record every plan

    # ------------------------------------------------------------------ requests

    def check(self, request: Request) -> None:
        """Raises for a request that could never run, before it takes a place in the line: only
        the offender is refused, whatever else is running."""
        if request.settings.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if not request.prompt:
            raise ValueError("prompt cannot be empty")
        if min(request.prompt) < 0 or max(request.prompt) >= self.runner.vocab_size:
            raise ValueError(f"request {request.request_id!r}: a prompt token is outside the vocabulary")
        longest = self.runner.cache.max_sequence_length
        if len(request.prompt) + request.settings.max_new_tokens > longest:
            raise RequestTooLongError(
                f"request {request.request_id!r}: {len(request.prompt)} prompt tokens and "
                f"{request.settings.max_new_tokens} new ones exceed the longest sequence, {longest}"
            )
        if request.request_id in self._known:
            raise ValueError(f"request {request.request_id!r} is already running")

    def submit(self, request: Request) -> None:
        self.check(request)
        self._known.add(request.request_id)
        self.scheduler.enqueue(request)

    @property
    def has_work(self) -> bool:
        return not self.scheduler.idle

    def finish(self, request: Request, error: Exception | None = None) -> None:
        """The request leaves the engine, with its tokens or with `error`; what it holds in the
        cache is given back (`engine.py:402-415`)."""
        self.scheduler.retire(request)
        if self.runner.has_request(request.request_id):
            self.runner.end_request(request.request_id)
        self._known.discard(request.request_id)
        self._evictions_of_finished += request.evictions
        self._replayed_by_finished += request.replayed_tokens
        request.error, request.done = error, True
        self.finished.append(request)

    def fail_all(self, error: Exception) -> None:
        """Everything running or waiting ends with `error` (`engine.py:417-426`)."""
        for request in self.scheduler.running + self.scheduler.waiting:
            self.finish(request, error)

    # ------------------------------------------------------------------ one iteration

    @staticmethod
    def _phase(batch: list[Request]) -> str:
        kinds = {request.in_prompt for request in batch}
        return "mixed" if len(kinds) == 2 else "prefill" if True in kinds else "decode"

    def step(self) -> list[TokenEvent]:
        """Admits, plans, makes room, runs one batch, samples (`engine.py:234-346`).
        Returns the tokens generated in this iteration."""
        for request in self.scheduler.admit():
            self.runner.add_request(request.request_id)
        batch = list(self.scheduler.running)
        if not batch:
            return []
        if not self.collect_iteration_metrics:
            return self._run_iteration(batch)
        phase = self._phase(batch)
        on_device = self.runner.device.type == "cuda"
        began = torch.cuda.Event(enable_timing=True) if on_device else None
        if began is not None:
            began.record()
        started = time.perf_counter()
        try:
            return self._run_iteration(batch)
        finally:
            self._host_ms[phase] += 1000.0 * (time.perf_counter() - started)
            self._iterations[phase] += 1
            if began is not None:
                ended = torch.cuda.Event(enable_timing=True)
                ended.record()
                self._device_spans[phase].append((began, ended))

    def _no_arrival_can_join(self, staying: list[Request]) -> bool:
        """Whether the next step's batch is certain to be `staying` unless a stop token comes: nobody
        waits, or nobody can be admitted (the batch stays full; a static batch is not empty)."""
        scheduler = self.scheduler
        if scheduler.num_waiting == 0:
            return True
        if scheduler.mode == "static":
            return bool(staying)
        return len(staying) == len(scheduler.running) == scheduler.limits.max_batch_size

    def _run_iteration(self, batch: list[Request]) -> list[TokenEvent]:
        in_flight, self._in_flight = self._in_flight, None
        if in_flight is not None and any(not request.done for request in in_flight.requests):
            # this iteration's step runs already: its requests each brought the token they had just been given
            rows = in_flight.requests
            logits = in_flight.logits
            shares = [Share(request, 1) for request in rows if not request.done]
            if self.step_log is not None:
                self.step_log.append([(request.request_id, 1) for request, _ in shares])
        else:
            expected, self._expected = self._expected, None
            if expected is not None and len(expected) == len(batch) and all(a is b for a, b in zip(expected, batch)):
                # the step that was prepared while the last one ran: every request brings the token it
                # has just been given, and the runner holds the cache entries already
                shares = [Share(request, 1) for request in batch]
            else:
                shares = self._plan()
                if not shares:
                    return []
            if self.step_log is not None:
                self.step_log.append([(request.request_id, count) for request, count in shares])
            entries, rows = [], []
            for request, count in shares:
                catches_up = count == request.owed  # else: a portion of a prompt, or of a replay after giving way
                entries.append(StepEntry(request.request_id, request.next_tokens(count), (count - 1,) if catches_up else ()))
                if catches_up:
                    rows.append(request)
            logits = self.runner.step(entries, fits_checked=True)
        for request, count in shares:
            request.cached += count
        if all(request.done for request in rows):
            return []
        settings = [request.settings for request in rows]
        draws = [len(request.output) for request in rows]
        tokens = None
        if self.look_ahead and len(rows) == len(shares) == len(batch) and not any(request.done for request in rows):
            # Every running request has just decoded: unless a stop token comes, the next step is these
            # requests again, less those at their last token.  The runner does its host work for that
            # step now, while the device is still busy with this one.
            staying = [request for request in rows if request.output_left > 1]
            if self._no_arrival_can_join(staying) and self.runner.prepare_decode([r.request_id for r in staying]):
                if self.run_ahead and len(staying) == len(rows):
                    # and queues it: the tokens go from the sampler to the step on the device
                    chosen = self.sampler.sample_on_device(logits, settings, draws)
                    fetch = self.runner.fetch_later(chosen)
                    next_logits = self.runner.step_from_device([r.request_id for r in staying], chosen)
                    self._in_flight = _StepInFlight(staying, next_logits)
                    tokens = fetch()
                else:
                    self._expected = staying
        if tokens is None:
            tokens = self.sampler.sample(logits, settings, draws)
        produced = []
        for request, token in zip(rows, tokens):
            if request.done:  # a row of a step queued before its request's end was known
                continue
            request.output.append(token)
            produced.append(TokenEvent(request, token))
            if request.output_left <= 0 or token in request.settings.stop_token_ids:
                self.finish(request)
        return produced

    def _plan(self) -> list[Share]:
        """Who brings how many tokens to this step.  A request that has outgrown the longest sequence
        ends alone, with an error of its own; when pages run out, requests give way (never the
        oldest) until the rest fits, and one that cannot fit even alone fails with `CacheFullError`."""
        shares = self.scheduler.plan(self.prefill_chunk_size)
        longest = self.runner.cache.max_sequence_length
        for request, count in shares:
            if request.cached + count > longest:  # `check` keeps such requests out; nobody else pays for one
                self.finish(request, RequestTooLongError(f"request {request.request_id!r} exceeds the longest sequence, {longest}"))
        shares = [share for share in shares if not share.request.done]

        def fits() -> bool:
            return self.runner.fits([(request.request_id, count) for request, count in shares])

        while len(shares) > 1 and not fits():
            victim = self.scheduler.victim(shares)
            self.runner.end_request(victim.request_id)
            self.scheduler.evict(victim)
            shares = [share for share in shares if share.request is not victim]
        if shares and not fits():
            self.finish(shares[0].request, CacheFullError("one sequence exceeds total KV cache capacity"))
            return []
        return shares

    # ------------------------------------------------------------------ synchronous use

    def generate(
        self,
        prompts: list[list[int]],
        configs: list[GenerationConfig] | GenerationConfig | None = None,
        request_ids: list[str] | None = None,
    ) -> list[list[int]]:
        """Runs the given prompts to completion and returns their generated tokens in order."""
        if configs is None or isinstance(configs, GenerationConfig):
            configs = [configs or GenerationConfig()] * len(prompts)
        names = request_ids or [f"request-{index:06d}" for index in range(len(prompts))]
        requests = [Request(name, list(prompt), config) for name, prompt, config in zip(names, prompts, configs)]
        for request in requests:
            self.submit(request)
        while self.has_work:
            self.step()
        failed = next((request for request in requests if request.error is not None), None)
        if failed is not None:
            raise failed.error
        return [request.output for request in requests]

    # ------------------------------------------------------------------ accounting

    @property
    def cache_stats(self) -> dict[str, float]:
        return self.runner.cache.stats(self.runner.cache.max_sequence_length)

    @property
    def iteration_stats(self) -> dict[str, float | int]:
        """The reference's keys (`engine.py:438-458`): iterations and host and device time by kind of
        iteration, what packing the steps' index arrays cost, and the evictions of finished requests."""
        stats: dict[str, float | int] = {
            "metadata_construction_ms": self.runner.packing_ms,
            "preemptions": self._evictions_of_finished,
            "recomputed_tokens": self._replayed_by_finished,
        }
        if any(self._device_spans.values()):
            torch.cuda.synchronize(self.runner.device)
        for how, count in getattr(self.runner, "step_counts", {}).items():
            stats[f"steps_{how}"] = count  # replayed from a graph, captured into one, launched kernel by kernel
        for phase in _PHASES:
            stats[f"{phase}_iterations"] = self._iterations[phase]
            stats[f"{phase}_cpu_ms"] = self._host_ms[phase]
            stats[f"{phase}_cuda_ms"] = sum(began.elapsed_time(ended) for began, ended in self._device_spans[phase])
        return stats


class LLMEngine:
    """The asynchronous entry point, with the reference's signature (`engine.py:108-242`).

    `model` is a model folder, or what `load_model_folder` returned.  `kernels`
    is the kernel library; by default the HIP library for `dtype` on `device`.
    Requests go into an inbox; one task serves them, an iteration at a time, and
    sleeps on an event while there is nothing to do.
    """

    def __init__(
        self,
        model: LoadedModel | str,
        tokenizer: Tokenizer | None = None,
        *,
        cache_config: CacheConfig | None = None,
        scheduler_config: SchedulerConfig | None = None,
        scheduler_mode: str = "continuous",
        prefill_chunk_size: int = 16,
        collect_iteration_metrics: bool = False,
        device: torch.device | str = "cuda:0",
        dtype: torch.dtype | str = torch.bfloat16,
        kernels: Any = None,
        max_sequence_length: int | None = None,
    ) -> None:
        from ..weights.loader import run_dtype

        dtype = run_dtype(dtype)
        if not isinstance(model, LoadedModel):
            model = load_model_folder(model, dtype)
        elif model.dtype != dtype:
            raise ValueError(f"the model was loaded as {model.dtype}, the engine is asked for {dtype}")
        if kernels is None:
            from ..kernels.hip import HipKernels

            kernels = HipKernels(dtype, device)
        self.tokenizer = tokenizer or ByteTokenizer()
        self.runner = ModelRunner(model, kernels, cache_config, max_sequence_length=max_sequence_length)
        self.core = EngineCore(
            self.runner,
            scheduler_config,
            scheduler_mode=scheduler_mode,
            prefill_chunk_size=prefill_chunk_size,
            collect_iteration_metrics=collect_iteration_metrics,
        )
        self.device = self.runner.device
        self._inbox: collections.deque[Request] = collections.deque()
        self._wake = asyncio.Event()
        self._server: asyncio.Task | None = None
        self._closed = False
        self._facts: dict[str, dict[str, float | int | None]] = {}  # in order of finishing
        self.facts_kept = 4096

    @property
    def scheduler(self) -> Scheduler:
        return self.core.scheduler

    @property
    def cache(self):
        return self.runner.cache

    async def generate(
        self,
        prompt: str | list[int],
        config: GenerationConfig | None = None,
        callback: TokenCallback | None = None,
        *,
        priority: int = 0,
        request_id: str | None = None,
    ) -> list[int]:
        """Generates for one prompt (text, or token ids) and returns the new tokens; `callback` gets
        each as it is produced.  A request that can never run is refused here, with `ValueError`."""
        if self._closed:
            raise RuntimeError("engine is closed")
        tokens = self.tokenizer.encode(prompt) if isinstance(prompt, str) else list(prompt)
        request = Request(request_id or uuid.uuid4().hex, tokens, config or GenerationConfig(), priority, callback)
        self.core.check(request)
        request.outcome = asyncio.get_running_loop().create_future()
        self._inbox.append(request)
        self._wake.set()
        if self._server is None or self._server.done():  # the first request, or the first after a step failed
            self._server = asyncio.create_task(self._serve())
        return await request.outcome

    def request_facts(self, request_id: str) -> dict[str, float | int | None]:
        """What the engine knows about a finished request beside its tokens: when it was first
        admitted (monotonic seconds), how often it gave way and how many tokens that cost.  Kept until
        asked for, the latest `facts_kept` requests at most."""
        return self._facts.pop(request_id, {})

    def _settle(self) -> None:
        """Hands every finished request's tokens, or its error, to whoever awaits it."""
        for request in self.core.finished:
            self._facts[request.request_id] = {
                "admitted_s": request.admitted_at,
                "preemptions": request.evictions,
                "recomputed_tokens": request.replayed_tokens,
            }
            while len(self._facts) > self.facts_kept:  # a caller that never asks does not make it grow
                del self._facts[next(iter(self._facts))]
            waiter = request.outcome
            if waiter is None or waiter.done():
                continue
            if request.error is None:
                waiter.set_result(request.output)
            else:
                waiter.set_exception(request.error)
        self.core.finished.clear()

    async def _serve(self) -> None:
        try:
            while True:
                while self._inbox:
                    request = self._inbox.popleft()
                    try:
                        self.core.submit(request)
                    except Exception as error:  # e.g. an id that is in use: only this request fails
                        request.outcome.set_exception(error)
                if not self.core.has_work:
                    self._wake.clear()
                    await self._wake.wait()
                    continue
                for event in self.core.step():
                    notify = event.request.on_token
                    if notify is not None:
                        pending = notify(event.token)
                        if inspect.isawaitable(pending):
                            await pending
                self._settle()
                await asyncio.sleep(0)  # callers run: new requests arrive, tokens are consumed
        except asyncio.CancelledError:
            raise
        except Exception as error:  # the step function failed: nobody can go on
            for request in self._inbox:
                request.outcome.set_exception(error)
            self._inbox.clear()
            self.core.fail_all(error)
            self._settle()

    async def close(self) -> None:
        """Stops serving and drops what the runner holds on the device beside the model (captured graphs)."""
        self._closed = True
        server, self._server = self._server, None
        if server is not None:
            server.cancel()
            await asyncio.gather(server, return_exceptions=True)
        self.runner.close()

    @property
    def cache_stats(self) -> dict[str, float]:
        return self.core.cache_stats

    @property
    def iteration_stats(self) -> dict[str, float | int]:
        return self.core.iteration_stats

    async def __aenter__(self) -> "LLMEngine":
        return self

    async def __aexit__(self, *_: Any) -> None:
        await self.close()
