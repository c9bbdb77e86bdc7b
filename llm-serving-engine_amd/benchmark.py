"""The open-loop benchmark: a seeded synthetic workload, a driver that sends each request at
its arrival time whatever the engine is doing, and a latency report.

What has to agree with the reference's harness (`src/llmserve/benchmark/{workload,metrics,runner}.py`)
does: the keys of a profile's YAML file, the order in which one seeded stream draws gaps, lengths
and token ids (`workload.py:60-79`: the same seed gives the same requests), the definitions of
time to first token, time per output token and end-to-end latency, percentiles by linear
interpolation, and the keys of the report's summary, so that reports can be laid side by side.
The rest is built around one table: a request's timeline is a row of plain values, the derived
columns are computed when the report is made, and summary, JSON and CSV are views of the rows.
"""

from __future__ import annotations

import asyncio
import csv
import dataclasses
import json
import math
import random
import time
from collections.abc import Awaitable, Callable, Iterator
from dataclasses import dataclass, field
from pathlib import Path


# --------------------------------------------------------------------------- the workload


@dataclass(frozen=True)
class LengthDistribution:
    """A log-normal length with the given median, rounded and clipped to [minimum, maximum]."""

    median: int
    sigma: float
    minimum: int
    maximum: int

    def draw(self, stream: random.Random) -> int:
        length = round(stream.lognormvariate(math.log(self.median), self.sigma))
        return max(self.minimum, min(length, self.maximum))

    def within(self, ceiling: int) -> "LengthDistribution":
        """The same distribution with both clips lowered to `ceiling` (at least 1)."""
        ceiling = max(1, ceiling)
        return dataclasses.replace(self, minimum=min(self.minimum, ceiling), maximum=min(self.maximum, ceiling))


@dataclass(frozen=True)
class RequestGroup:
    """A run of consecutive requests with length distributions of their own."""

    requests: int
    prompt: LengthDistribution
    output: LengthDistribution


@dataclass(frozen=True)
class Arrival:
    """One request of the workload: when it is sent, what it brings and how much it asks for."""

    request_id: str
    at_s: float
    prompt: tuple[int, ...]
    max_new_tokens: int


@dataclass(frozen=True)
class LoadProfile:
    """A profile file's keys (configs/benchmark-sharegpt.yaml; defaults as `workload.py:25-46`).
    `groups`, which the reference does not have, makes a mix: the first group's requests arrive
    first, then the second's, all on the one arrival process; `requests` is then their total."""

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

    @classmethod
    def from_yaml(cls, path: str | Path) -> "LoadProfile":
        import yaml

        values = yaml.safe_load(Path(path).read_text())
        fields = {}
        for key in ("arrival_rate", "seed", "vocabulary_size"):
            if key in values:
                fields[key] = values[key]
        for key in ("prompt", "output"):
            if key in values:
                fields[key] = LengthDistribution(**values[key])
        if "groups" in values:
            fields["groups"] = tuple(
                RequestGroup(item["requests"], LengthDistribution(**item["prompt"]), LengthDistribution(**item["output"]))
                for item in values["groups"]
            )
            fields["requests"] = sum(group.requests for group in fields["groups"])
        if "requests" in values:
            fields["requests"] = values["requests"]
        if "arrival_rate" not in fields:
            raise ValueError(f"{path}: a profile needs arrival_rate")
        return cls(**fields)

    def to_dict(self) -> dict[str, object]:
        return dataclasses.asdict(self)

    def fitted(self, longest_sequence: int) -> "LoadProfile":
        """The same profile with prompts clipped so that prompt plus output fit `longest_sequence`."""
        groups = tuple(
            dataclasses.replace(group, prompt=group.prompt.within(longest_sequence - group.output.maximum))
            for group in self.groups
        )
        return dataclasses.replace(self, prompt=self.prompt.within(longest_sequence - self.output.maximum), groups=groups)

    def _lengths(self) -> Iterator[tuple[LengthDistribution, LengthDistribution]]:
        if not self.groups:
            for _ in range(self.requests):
                yield self.prompt, self.output
        for group in self.groups:
            for _ in range(group.requests):
                yield group.prompt, group.output

    def arrivals(self) -> list[Arrival]:
        """The workload.  One seeded stream draws, per request and in this order: the gap since the
        previous arrival (exponential; none before the first), the prompt's length, the output's
        length, then the prompt's token ids, uniform over the vocabulary less the reserved ids 0-3."""
        if self.arrival_rate <= 0:
            raise ValueError("arrival_rate must be positive")
        stream = random.Random(self.seed)
        clock = 0.0
        workload = []
        for prompts, outputs in self._lengths():
            if workload:
                clock += stream.expovariate(self.arrival_rate)
            prompt_length, wanted = prompts.draw(stream), outputs.draw(stream)
            prompt = tuple(stream.randrange(4, self.vocabulary_size) for _ in range(prompt_length))
            workload.append(Arrival(f"request-{len(workload):06d}", clock, prompt, wanted))
        return workload


def generate_workload(profile: LoadProfile) -> list[Arrival]:
    return profile.arrivals()


# --------------------------------------------------------------------------- the report


def percentile(values: list[float], quantile: float) -> float:
    """The `quantile` point of `values` by linear interpolation between neighbours in sorted order
    (0.0 for no values), as `metrics.py:11-21` defines it."""
    if not values:
        return 0.0
    ranked = sorted(values)
    place = quantile * (len(ranked) - 1)
    below = int(place)
    above = min(below + 1, len(ranked) - 1)
    return ranked[below] + (place - below) * (ranked[above] - ranked[below])


def _span_ms(begin: float | None, end: float | None) -> float | None:
    return None if begin is None or end is None else (end - begin) * 1000.0


@dataclass
class RequestMetrics:
    """One request's timeline; times are seconds on one monotonic clock.  `admitted_s`,
    `preemptions` and `recomputed_tokens` come from the engine where it reports them
    (`metrics.py:29,33-34` has the fields)."""

    request_id: str
    arrival_s: float
    prompt_tokens: int
    requested_output_tokens: int
    admitted_s: float | None = None
    first_token_s: float | None = None
    finished_s: float | None = None
    output_tokens: int = 0
    preemptions: int = 0
    recomputed_tokens: int = 0
    error: str | None = None

    @property
    def ttft_ms(self) -> float | None:
        """Arrival to first token."""
        return _span_ms(self.arrival_s, self.first_token_s)

    @property
    def tpot_ms(self) -> float | None:
        """First token to last, per token after the first; None for fewer than two tokens."""
        whole = _span_ms(self.first_token_s, self.finished_s)
        return None if whole is None or self.output_tokens < 2 else whole / (self.output_tokens - 1)

    @property
    def e2e_ms(self) -> float | None:
        """Arrival to the end."""
        return _span_ms(self.arrival_s, self.finished_s)

    def to_dict(self) -> dict[str, object]:
        row = dataclasses.asdict(self)
        for column in LATENCIES:
            row[column] = getattr(self, column)
        return row


LATENCIES = ("ttft_ms", "tpot_ms", "e2e_ms")
QUANTILES = {"p50": 0.50, "p95": 0.95, "p99": 0.99}


@dataclass
class BenchmarkReport:
    config_name: str
    started_s: float
    finished_s: float
    requests: list[RequestMetrics]
    cache: dict[str, float] = field(default_factory=dict)
    metadata: dict[str, object] = field(default_factory=dict)

    def rows(self) -> list[dict[str, object]]:
        return [record.to_dict() for record in self.requests]

    @property
    def summary(self) -> dict[str, object]:
        """Counts, throughput (output tokens of successful requests over wall time), the latency
        percentiles of successful requests and the cache's figures; keys as `metrics.py:71-94`."""
        rows = [row for row in self.rows() if row["error"] is None]
        wall = max(self.finished_s - self.started_s, 1e-9)
        summary: dict[str, object] = {
            "config": self.config_name,
            "requests": len(self.requests),
            "successful_requests": len(rows),
            "duration_s": wall,
            "throughput_tokens_per_s": sum(row["output_tokens"] for row in rows) / wall,
            "preemptions": sum(row["preemptions"] for row in rows),
            "recomputed_tokens": sum(row["recomputed_tokens"] for row in rows),
        }
        for column in LATENCIES:
            known = [row[column] for row in rows if row[column] is not None]
            for label, quantile in QUANTILES.items():
                summary[f"{column}_{label}"] = percentile(known, quantile)
        for key, value in self.cache.items():
            summary[f"cache_{key}"] = value
        return summary

    def write_json(self, path: str | Path) -> None:
        document = {"summary": self.summary, "metadata": self.metadata, "requests": self.rows()}
        Path(path).write_text(json.dumps(document, indent=2) + "\n")

    def write_csv(self, path: str | Path) -> None:
        rows = self.rows()
        if not rows:
            return
        with Path(path).open("w", newline="") as handle:
            table = csv.DictWriter(handle, fieldnames=list(rows[0]))
            table.writeheader()
            table.writerows(rows)


# --------------------------------------------------------------------------- the driver

Generate = Callable[[Arrival, Callable[[int], None]], Awaitable[list[int]]]
Facts = Callable[[str], dict]


class BenchmarkHarness:
    """Open loop: a dispatcher walks the arrivals in time order, sleeps until each is due and
    starts it as a task of its own, so a slow engine delays nobody's arrival; every request's
    first and last token are timed on the monotonic clock."""

    def __init__(self, profile: LoadProfile) -> None:
        self.profile = profile
        self.workload = profile.arrivals()

    async def run(self, name: str, generate: Generate, facts: Facts | None = None) -> BenchmarkReport:
        """`generate(arrival, on_token)` serves one request; `facts(request_id)`, if given, returns what
        the engine knows about a finished request (`admitted_s`, `preemptions`, `recomputed_tokens`)."""
        clock = time.monotonic
        origin = clock()
        records: dict[str, RequestMetrics] = {}

        async def serve(arrival: Arrival) -> None:
            record = RequestMetrics(arrival.request_id, clock(), len(arrival.prompt), arrival.max_new_tokens)
            records[arrival.request_id] = record

            def on_token(_: int) -> None:
                record.output_tokens += 1
                if record.output_tokens == 1:
                    record.first_token_s = clock()

            try:
                await generate(arrival, on_token)
            except Exception as error:  # a failed request is a row of the report; the run goes on
                record.error = f"{type(error).__name__}: {error}"
            record.finished_s = clock()
            if facts is not None:
                for key, value in facts(arrival.request_id).items():
                    setattr(record, key, value)

        in_service = []
        for arrival in self.workload:
            wait = origin + arrival.at_s - clock()
            if wait > 0:
                await asyncio.sleep(wait)
            in_service.append(asyncio.create_task(serve(arrival)))
        if in_service:
            await asyncio.wait(in_service)
        ordered = [records[arrival.request_id] for arrival in self.workload]
        return BenchmarkReport(name, origin, clock(), ordered, metadata={"profile": self.profile.to_dict()})
