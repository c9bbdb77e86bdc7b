"""The engine above the step function: it admits requests, plans each
iteration, makes room when pages run out, samples, streams and finishes.

`EngineCore` is the synchronous loop body (one call of `step()` is one
iteration).  `LLMEngine` is the asynchronous entry point with the reference's
interface (`engine.py:108-464`): `await engine.generate(prompt, config,
callback, priority=, request_id=)`.
"""

from __future__ import annotations

import asyncio
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
from .scheduler import IterationScheduler, RequestState, TokenCallback, choose_victim, plan_iteration
from .tokenizer import ByteTokenizer, Tokenizer


@dataclass
class TokenEvent:
    request: RequestState
    token: int


@dataclass
class _StepInFlight:
    """A decode step that was queued before the tokens it consumes had reached the host."""

    requests: list[RequestState]  # row i of `logits` is requests[i]
    logits: torch.Tensor


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
        scheduler_config = scheduler_config or SchedulerConfig()
        if prefill_chunk_size <= 0:
            raise ValueError("prefill_chunk_size must be positive")
        if scheduler_config.max_tokens_per_step < scheduler_config.max_batch_size:
            raise ValueError("max_tokens_per_step must allow one token per active request")
        if scheduler_config.max_batch_size > runner.cache_config.max_sequences:
            raise ValueError("max_batch_size exceeds the cache's request slots (CacheConfig.max_sequences)")
        self.runner = runner
        self.scheduler_config = scheduler_config
        self.scheduler = IterationScheduler(scheduler_config.max_batch_size, scheduler_config.policy, scheduler_mode)
        self.prefill_chunk_size = prefill_chunk_size
        self.sampler = Sampler(runner.kernels)
        self.collect_iteration_metrics = collect_iteration_metrics
        self.look_ahead = look_ahead  # prepare the next decode step on the host while the device runs this one
        self._expected: list[RequestState] | None = None  # the requests of the step that is prepared
        # Queue the next decode step behind the sampling of this one, its tokens passed on the device:
        # the device then never waits for the host between two steps.  A request that turns out to have
        # ended (a stop token) has a row in that step that nobody reads.
        self.run_ahead = run_ahead and look_ahead
        self._in_flight: _StepInFlight | None = None
        self.generation_configs: dict[str, GenerationConfig] = {}
        self.finished: list[RequestState] = []
        self._cpu_ms = {"prefill": 0.0, "decode": 0.0, "mixed": 0.0}
        self._counts = {"prefill": 0, "decode": 0, "mixed": 0}
        self._events: dict[str, list] = {"prefill": [], "decode": [], "mixed": []}
        self._completed_preemptions = 0
        self._completed_recomputed_tokens = 0
        self.step_log: list[list[tuple[str, int]]] | None = None  # tests set it to [] to record every plan

    # ------------------------------------------------------------------ requests

    def submit(self, request: RequestState, config: GenerationConfig) -> None:
        if config.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if not request.prompt_token_ids:
            raise ValueError("prompt cannot be empty")
        if request.request_id in self.generation_configs:
            raise ValueError(f"request {request.request_id!r} is already running")
        self.generation_configs[request.request_id] = config
        self.scheduler.add(request)

    @property
    def has_work(self) -> bool:
        return not self.scheduler.empty

    def finish(self, request: RequestState, error: Exception | None = None) -> None:
        """`engine.py:402-415`."""
        if request in self.scheduler.active:
            self.scheduler.finish(request)
        if request in self.scheduler.waiting:
            self.scheduler.waiting.remove(request)
        if self.runner.has_request(request.request_id):
            self.runner.end_request(request.request_id)
        self.generation_configs.pop(request.request_id, None)
        self._completed_preemptions += request.preemptions
        self._completed_recomputed_tokens += request.recomputed_tokens
        request.error = error
        request.finished = True
        self.finished.append(request)

    def fail_all(self, error: Exception) -> None:
        """`engine.py:417-426`."""
        for request in list(self.scheduler.active) + list(self.scheduler.waiting):
            self.finish(request, error)

    # ------------------------------------------------------------------ one iteration

    @staticmethod
    def _phase(active: list[RequestState]) -> str:
        prefill = any(request.in_prefill for request in active)
        decode = any(not request.in_prefill for request in active)
        return "mixed" if prefill and decode else "prefill" if prefill else "decode"

    def step(self) -> list[TokenEvent]:
        """Admits, plans, makes room, runs one batch, samples (`engine.py:234-346`).
        Returns the tokens generated in this iteration."""
        for request in self.scheduler.admit():
            self.runner.add_request(request.request_id)
        active = list(self.scheduler.active)
        if not active:
            return []
        phase = self._phase(active)
        started = time.perf_counter()
        events = None
        if self.collect_iteration_metrics and self.runner.device.type == "cuda":
            events = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            events[0].record()
        try:
            return self._run_iteration(active)
        finally:
            if self.collect_iteration_metrics:
                self._cpu_ms[phase] += (time.perf_counter() - started) * 1000
                self._counts[phase] += 1
                if events is not None:
                    events[1].record()
                    self._events[phase].append(events)

    def _run_iteration(self, active: list[RequestState]) -> list[TokenEvent]:
        in_flight, self._in_flight = self._in_flight, None
        if in_flight is not None and any(not request.finished for request in in_flight.requests):
            # this iteration's step runs already: its requests each brought the token they had just been given
            rows = in_flight.requests
            logits = in_flight.logits
            planned = [(request, 1) for request in rows if not request.finished]
            if self.step_log is not None:
                self.step_log.append([(request.request_id, 1) for request, _ in planned])
        else:
            expected, self._expected = self._expected, None
            if expected is not None and len(expected) == len(active) and all(a is b for a, b in zip(expected, active)):
                # the step that was prepared while the last one ran: every request brings the token it
                # has just been given, and the runner holds the cache entries already
                planned = [(request, 1) for request in active]
            else:
                planned = self._plan(active)
                if planned is None:
                    return []
            if self.step_log is not None:
                self.step_log.append([(request.request_id, count) for request, count in planned])

            entries, rows = [], []
            for request, count in planned:
                tokens = request.tokens_between(request.processed_tokens, request.processed_tokens + count)
                last = request.processed_tokens + count == len(request.prompt_token_ids) + len(request.generated_token_ids)
                entries.append(StepEntry(request.request_id, tokens, (count - 1,) if last else ()))
                if last:  # otherwise: a portion of a prompt, or a replay after preemption
                    rows.append(request)
            logits = self.runner.step(entries, fits_checked=True)
        for request, count in planned:
            request.processed_tokens += count
        sampled = [request for request in rows if not request.finished]
        if not sampled:
            return []
        greedy = GenerationConfig()
        configs = [self.generation_configs.get(request.request_id, greedy) for request in rows]
        steps = [len(request.generated_token_ids) for request in rows]
        tokens = None
        if self.look_ahead and len(sampled) == len(rows) == len(planned) == len(active) and not self.scheduler.waiting:
            # Every running request has just decoded and nothing waits: unless a stop token comes,
            # the next step is these requests again, less those at their last token.  The runner does
            # its host work for that step now, while the device is still busy with this one.
            staying = [r for r in sampled if len(r.generated_token_ids) + 1 < r.max_new_tokens]
            if self.runner.prepare_decode([r.request_id for r in staying]):
                if self.run_ahead and len(staying) == len(rows):
                    # and queues it: the tokens go from the sampler to the step on the device
                    chosen = self.sampler.sample_on_device(logits, configs, steps)
                    fetch = self.runner.fetch_later(chosen)
                    next_logits = self.runner.step_from_device([r.request_id for r in staying], chosen)
                    self._in_flight = _StepInFlight(staying, next_logits)
                    tokens = fetch()
                else:
                    self._expected = staying
        if tokens is None:
            tokens = self.sampler.sample(logits, configs, steps)
        produced = []
        for request, config, token in zip(rows, configs, tokens):
            if request.finished:  # a row of a step queued before its request's end was known
                continue
            request.generated_token_ids.append(token)
            produced.append(TokenEvent(request, token))
            if len(request.generated_token_ids) >= request.max_new_tokens or token in config.stop_token_ids:
                self.finish(request)
        return produced

    def _plan(self, active: list[RequestState]) -> list[tuple[RequestState, int]] | None:
        """Who brings how many tokens to this step; requests give way until it fits the cache."""
        planned = plan_iteration(active, self.scheduler_config.max_tokens_per_step, self.prefill_chunk_size)

        def as_plan(items):
            return [(request.request_id, count) for request, count in items]

        # Pages run out: requests give way (never the oldest) until the rest fits.
        while not self.runner.fits(as_plan(planned)) and len(planned) > 1:
            victim = choose_victim(planned, self.scheduler_config.preemption)
            self.runner.end_request(victim.request_id)
            self.scheduler.preempt(victim)
            planned = [item for item in planned if item[0] is not victim]
        if not self.runner.fits(as_plan(planned)):
            self.finish(planned[0][0], CacheFullError("one sequence exceeds total KV cache capacity"))
            return None
        return planned

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
        requests = []
        for index, (prompt, config) in enumerate(zip(prompts, configs)):
            request_id = request_ids[index] if request_ids else f"request-{index:06d}"
            request = RequestState(request_id, list(prompt), config.max_new_tokens)
            self.submit(request, config)
            requests.append(request)
        while self.has_work:
            self.step()
        for request in requests:
            if request.error is not None:
                raise request.error
        return [request.generated_token_ids for request in requests]

    # ------------------------------------------------------------------ accounting

    @property
    def cache_stats(self) -> dict[str, float]:
        return self.runner.cache.stats(self.runner.cache.max_sequence_length)

    @property
    def iteration_stats(self) -> dict[str, float | int]:
        """`engine.py:438-458`."""
        device_ms = {phase: 0.0 for phase in self._events}
        if self.collect_iteration_metrics and self.runner.device.type == "cuda":
            torch.cuda.synchronize(self.runner.device)
            device_ms = {
                phase: sum(start.elapsed_time(end) for start, end in pairs) for phase, pairs in self._events.items()
            }
        result: dict[str, float | int] = {
            "preemptions": self._completed_preemptions,
            "recomputed_tokens": self._completed_recomputed_tokens,
        }
        for phase in ("prefill", "decode", "mixed"):
            result[f"{phase}_iterations"] = self._counts[phase]
            result[f"{phase}_cpu_ms"] = self._cpu_ms[phase]
            result[f"{phase}_cuda_ms"] = device_ms[phase]
        return result


class LLMEngine:
    """Asynchronous iteration-level engine (`engine.py:108-242`).

    `model` is a model folder, or what `load_model_folder` returned.  `kernels`
    is the kernel library; by default the HIP library for `dtype` on `device`.
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
        paged_attention_backend: str = "hip",
        cache_device_metadata: bool = True,
    ) -> None:
        """`paged_attention_backend` and `cache_device_metadata` are the reference's switches between its own
        back ends (`engine.py:111-125`), taken so that its calls carry over: there is one attention path here
        (the reference's names "pytorch" and "triton" are read as it), and a step's index arrays are packed
        anew for every step whatever the second says."""
        from ..weights.loader import run_dtype

        if paged_attention_backend not in ("hip", "pytorch", "triton"):
            raise ValueError(f"unknown paged_attention_backend {paged_attention_backend!r}")
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
        self._incoming: asyncio.Queue[RequestState] = asyncio.Queue()
        self._worker: asyncio.Task | None = None
        self._closed = False
        self._pending_configs: dict[str, GenerationConfig] = {}

    @property
    def scheduler(self) -> IterationScheduler:
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
        """`engine.py:188-221`."""
        config = config or GenerationConfig()
        if self._closed:
            raise RuntimeError("engine is closed")
        if config.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if self._worker is None:
            self._worker = asyncio.create_task(self._run())
        prompt_tokens = self.tokenizer.encode(prompt) if isinstance(prompt, str) else list(prompt)
        if not prompt_tokens:
            raise ValueError("prompt cannot be empty")
        request_id = request_id or str(uuid.uuid4())
        future = asyncio.get_running_loop().create_future()
        state = RequestState(
            request_id=request_id,
            prompt_token_ids=prompt_tokens,
            max_new_tokens=config.max_new_tokens,
            callback=callback,
            priority=priority,
            future=future,
        )
        self._pending_configs[request_id] = config
        await self._incoming.put(state)
        return await future

    def _take(self, request: RequestState) -> None:
        try:
            self.core.submit(request, self._pending_configs.pop(request.request_id))
        except Exception as error:
            if request.future and not request.future.done():
                request.future.set_exception(error)

    async def _run(self) -> None:
        """`engine.py:223-242`."""
        try:
            while not self._closed:
                if not self.core.has_work:
                    self._take(await self._incoming.get())
                while True:
                    try:
                        self._take(self._incoming.get_nowait())
                    except asyncio.QueueEmpty:
                        break
                events = self.core.step()
                for event in events:
                    if event.request.callback:
                        result = event.request.callback(event.token)
                        if inspect.isawaitable(result):
                            await result
                self._resolve()
                await asyncio.sleep(0)
        except asyncio.CancelledError:
            pass
        except Exception as error:
            self.core.fail_all(error)
            self._resolve()

    def _resolve(self) -> None:
        for request in self.core.finished:
            if request.future and not request.future.done():
                if request.error is not None:
                    request.future.set_exception(request.error)
                else:
                    request.future.set_result(request.generated_token_ids)
        self.core.finished.clear()

    async def close(self) -> None:
        self._closed = True
        if self._worker:
            self._worker.cancel()
            await asyncio.gather(self._worker, return_exceptions=True)

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
