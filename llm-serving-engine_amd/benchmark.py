"""The synthetic workload and the latency metrics of the reference's benchmark harness
(`src/llmserve/benchmark/{workload,metrics,runner}.py`), restated: clipped log-normal prompt
and output lengths, exponential gaps between arrivals, uniform token ids, everything fixed by
one seed; time to first token, time per output token, end-to-end latency, tokens per second.
"""

from __future__ import annotations

import asyncio
import csv
import json
import math
import random
import time
from dataclasses import asdict, dataclass, field
from pathlib import Path
from typing import Awaitable, Callable


@dataclass(frozen=True)
class LengthDistribution:
    """round(lognormal(ln median, sigma)) clipped to [minimum, maximum] (`workload.py:11-22`)."""

    median: int
    sigma: float
    minimum: int
    maximum: int

    def sample(self, rng: random.Random) -> int:
        drawn = round(rng.lognormvariate(math.log(self.median), self.sigma))
        return min(self.maximum, max(self.minimum, drawn))


@dataclass(frozen=True)
class RequestGroup:
    """A run of consecutive requests with length distributions of their own."""

    requests: int
    prompt: LengthDistribution
    output: LengthDistribution


@dataclass(frozen=True)
class LoadProfile:
    """`workload.py:25-46` and configs/benchmark-sharegpt.yaml.  `groups`, which the reference
    does not have, makes a mix: the first group's requests arrive first, then the second's, all
    on the one arrival process; `requests` is then the groups' total."""

    requests: int = 100
    arrival_rate: float = 2.0
    prompt: LengthDistribution = LengthDistribution(128, 0.9, 8, 1_024)
    output: LengthDistribution = LengthDistribution(64, 0.7, 4, 256)
    seed: int = 7
    vocabulary_size: int = 32_000
    groups: tuple[RequestGroup, ...] = ()

    def __post_init__(self) -> None:
        if self.groups and sum(group.requests for group in self.groups) != self.requests:
            raise ValueError("requests must be the sum of the groups' requests")

    def distributions(self) -> list[tuple[LengthDistribution, LengthDistribution]]:
        """(prompt, output) distributions of every request, in arrival order."""
        if not self.groups:
            return [(self.prompt, self.output)] * self.requests
        return [(group.prompt, group.output) for group in self.groups for _ in range(group.requests)]

    def fitted(self, longest_sequence: int) -> "LoadProfile":
        """The same profile with prompts clipped so that prompt plus output fit `longest_sequence`."""
        from dataclasses import replace

        def clip(prompt: LengthDistribution, output: LengthDistribution) -> LengthDistribution:
            return replace(prompt, maximum=max(1, min(prompt.maximum, longest_sequence - output.maximum)),
                           minimum=max(1, min(prompt.minimum, longest_sequence - output.maximum)))

        groups = tuple(replace(group, prompt=clip(group.prompt, group.output)) for group in self.groups)
        return replace(self, prompt=clip(self.prompt, self.output), groups=groups)

    @classmethod
    def from_yaml(cls, path: str | Path) -> "LoadProfile":
        import yaml

        with Path(path).open() as handle:
            values = yaml.safe_load(handle)
        groups = tuple(
            RequestGroup(group["requests"], LengthDistribution(**group["prompt"]), LengthDistribution(**group["output"]))
            for group in values.get("groups", ())
        )
        defaults = cls()
        return cls(
            requests=values.get("requests", sum(group.requests for group in groups) or defaults.requests),
            arrival_rate=values["arrival_rate"],
            prompt=LengthDistribution(**values["prompt"]) if "prompt" in values else defaults.prompt,
            output=LengthDistribution(**values["output"]) if "output" in values else defaults.output,
            seed=values.get("seed", 7),
            vocabulary_size=values.get("vocabulary_size", 32_000),
            groups=groups,
        )

    def to_dict(self) -> dict[str, object]:
        return asdict(self)


@dataclass(frozen=True)
class RequestSpec:
    request_id: str
    arrival_offset_s: float
    prompt_token_ids: tuple[int, ...]
    max_new_tokens: int


def generate_workload(profile: LoadProfile) -> list[RequestSpec]:
    """One seeded stream draws, per request, the gap to the previous arrival (none for the
    first), the prompt length, the output length and the prompt's token ids, which avoid
    the reserved ids 0-3 (`workload.py:60-79`)."""
    if profile.arrival_rate <= 0:
        raise ValueError("arrival_rate must be positive")
    rng = random.Random(profile.seed)
    at = 0.0
    specs = []
    for index, (prompt_lengths, output_lengths) in enumerate(profile.distributions()):
        if index:
            at += rng.expovariate(profile.arrival_rate)
        prompt_length = prompt_lengths.sample(rng)
        output_length = output_lengths.sample(rng)
        prompt = tuple(rng.randrange(4, profile.vocabulary_size) for _ in range(prompt_length))
        specs.append(RequestSpec(f"request-{index:06d}", at, prompt, output_length))
    return specs


def percentile(values: list[float], quantile: float) -> float:
    """Linear interpolation between order statistics (`metrics.py:11-21`)."""
    if not values:
        return 0.0
    ordered = sorted(values)
    where = (len(ordered) - 1) * quantile
    low, high = math.floor(where), math.ceil(where)
    return ordered[low] + (ordered[high] - ordered[low]) * (where - low)


@dataclass
class RequestMetrics:
    """Times are seconds on one monotonic clock (`metrics.py:24-58`)."""

    request_id: str
    arrival_s: float
    prompt_tokens: int
    requested_output_tokens: int
    first_token_s: float | None = None
    finished_s: float | None = None
    output_tokens: int = 0
    error: str | None = None

    @property
    def ttft_ms(self) -> float | None:
        return None if self.first_token_s is None else 1000 * (self.first_token_s - self.arrival_s)

    @property
    def tpot_ms(self) -> float | None:
        if self.first_token_s is None or self.finished_s is None or self.output_tokens < 2:
            return None
        return 1000 * (self.finished_s - self.first_token_s) / (self.output_tokens - 1)

    @property
    def e2e_ms(self) -> float | None:
        return None if self.finished_s is None else 1000 * (self.finished_s - self.arrival_s)

    def to_dict(self) -> dict[str, object]:
        return {**asdict(self), "ttft_ms": self.ttft_ms, "tpot_ms": self.tpot_ms, "e2e_ms": self.e2e_ms}


@dataclass
class BenchmarkReport:
    config_name: str
    started_s: float
    finished_s: float
    requests: list[RequestMetrics]
    cache: dict[str, float] = field(default_factory=dict)
    metadata: dict[str, object] = field(default_factory=dict)

    @property
    def summary(self) -> dict[str, object]:
        """`metrics.py:71-94`: throughput is output tokens of successful requests over wall time."""
        good = [item for item in self.requests if item.error is None]
        duration = max(self.finished_s - self.started_s, 1e-9)
        result: dict[str, object] = {
            "config": self.config_name,
            "requests": len(self.requests),
            "successful_requests": len(good),
            "duration_s": duration,
            "throughput_tokens_per_s": sum(item.output_tokens for item in good) / duration,
        }
        for name in ("ttft_ms", "tpot_ms", "e2e_ms"):
            values = [getattr(item, name) for item in good if getattr(item, name) is not None]
            for label, quantile in (("p50", 0.5), ("p95", 0.95), ("p99", 0.99)):
                result[f"{name}_{label}"] = percentile(values, quantile)
        result.update({f"cache_{key}": value for key, value in self.cache.items()})
        return result

    def write_json(self, path: str | Path) -> None:
        payload = {"summary": self.summary, "metadata": self.metadata, "requests": [r.to_dict() for r in self.requests]}
        Path(path).write_text(json.dumps(payload, indent=2) + "\n")

    def write_csv(self, path: str | Path) -> None:
        rows = [item.to_dict() for item in self.requests]
        if rows:
            with Path(path).open("w", newline="") as handle:
                writer = csv.DictWriter(handle, fieldnames=list(rows[0]))
                writer.writeheader()
                writer.writerows(rows)


Generate = Callable[[RequestSpec, Callable[[int], None]], Awaitable[list[int]]]


class BenchmarkHarness:
    """Open loop: every request is sent at its arrival offset whatever the engine is doing
    (`runner.py`), and its first and last token are timed."""

    def __init__(self, profile: LoadProfile) -> None:
        self.profile = profile
        self.workload = generate_workload(profile)

    async def run(self, name: str, generate: Generate) -> BenchmarkReport:
        started = time.monotonic()
        metrics: list[RequestMetrics] = []

        async def one(spec: RequestSpec) -> None:
            await asyncio.sleep(max(0.0, started + spec.arrival_offset_s - time.monotonic()))
            record = RequestMetrics(spec.request_id, time.monotonic(), len(spec.prompt_token_ids), spec.max_new_tokens)
            metrics.append(record)

            def on_token(_: int) -> None:
                if record.first_token_s is None:
                    record.first_token_s = time.monotonic()
                record.output_tokens += 1

            try:
                await generate(spec, on_token)
            except Exception as error:  # a failed request is reported, the run goes on
                record.error = f"{type(error).__name__}: {error}"
            record.finished_s = time.monotonic()

        await asyncio.gather(*(one(spec) for spec in self.workload))
        metrics.sort(key=lambda item: item.request_id)
        report = BenchmarkReport(name, started, time.monotonic(), metrics)
        report.metadata["profile"] = self.profile.to_dict()
        return report
