"""Cache and scheduler options, with the reference's names and defaults
(`src/llmserve/config.py:65-76`)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class CacheConfig:
    block_size: int = 16  # tokens per page
    num_blocks: int = 1_024  # pages in each group's pool
    max_sequences: int = 256  # live requests (block-table rows and state slots)

    def __post_init__(self) -> None:
        if self.block_size <= 0 or self.num_blocks <= 0 or self.max_sequences <= 0:
            raise ValueError("block_size, num_blocks and max_sequences must be positive")


@dataclass(frozen=True)
class SchedulerConfig:
    max_batch_size: int = 16
    max_tokens_per_step: int = 2_048
    policy: str = "fcfs"  # fcfs | sjf | priority
    preemption: str = "largest"  # who gives way when pages run out: largest | latest (never the oldest)
