"""Greedy, temperature and top-p sampling (reference `engine.py:20-72`).

Options and their meanings are the reference's.  What differs is where the
randomness comes from: the reference draws with `torch.multinomial` from a
generator per request; here each draw is one uniform number that depends only
on the request's seed and on how many tokens it has sampled so far, and the
kernel inverts the distribution's CDF at it.  A request therefore samples the
same tokens whatever else is in the batch and whether or not it was preempted.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class GenerationConfig:
    """`engine.py:20-26`."""

    max_new_tokens: int = 32
    temperature: float = 0.0
    top_p: float = 1.0
    seed: int = 7
    stop_token_ids: tuple[int, ...] = ()


_MASK = (1 << 64) - 1


def uniform_for(seed: int, step: int) -> float:
    """A float32-exact number in [0, 1): the top 24 bits of splitmix64(seed * 2^32 + step)."""
    z = (((seed & 0xFFFFFFFF) << 32) | (step & 0xFFFFFFFF)) & _MASK
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


class Sampler:
    """Chooses one token per row of logits with the kernel library's sampling kernels."""

    def __init__(self, kernels) -> None:
        self.kernels = kernels

    def sample(self, logits: torch.Tensor, configs: list[GenerationConfig], steps: list[int]) -> list[int]:
        """`steps[i]` is the number of tokens row i's request has sampled before.
        One device-to-host copy for the whole batch (`engine.py:44-72`)."""
        return self.sample_on_device(logits, configs, steps).cpu().tolist()

    def sample_on_device(self, logits: torch.Tensor, configs: list[GenerationConfig], steps: list[int]) -> torch.Tensor:
        """The same, left on the device as an integer tensor [rows]: nothing waits for the result."""
        if logits.ndim != 2 or logits.shape[0] != len(configs) or len(configs) != len(steps):
            raise ValueError("batched sampling inputs must have matching rows")
        if all(config.temperature <= 0 for config in configs):
            return self.kernels.argmax(logits)
        values = torch.tensor(
            [
                [config.temperature for config in configs],
                [config.top_p for config in configs],
                [uniform_for(config.seed, step) for config, step in zip(configs, steps)],
            ],
            dtype=torch.float32,
        )
        values = self.kernels.queued_to_device(values)
        with_top_p = any(config.temperature > 0 and config.top_p < 1 for config in configs)
        return self.kernels.sample(logits, values[0], values[1], values[2], with_top_p)
