"""What every part of a layer has in common: a spec (its sizes and constants),
the tensors it owns by name, what it needs of the cache, and a registry that
maps a spec's `kind` to the class that runs it.

A part never sees a model configuration.  It is built from its own spec, the
tensors under its own prefix and the kernel library, so a model may use
different mixers and feed-forwards in different layers, and a new part is added
by registering a class: nothing else changes.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

import torch


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part owns.

    role decides how the random-weights mode draws it: "matrix" and "embedding"
    N(0, std), "bias" N(0, bias_std), "norm" N(1, norm_std) (ones when
    norm_std is 0), "table" integers.  `integer` tensors are kept as int32; the
    others in the run's dtype unless the file stores them in 32-bit.
    """

    shape: tuple[int, ...]
    role: str = "matrix"
    integer: bool = False


@dataclass(frozen=True)
class PagedKeyValue:
    """Cache need of a mixer that keeps a key and a value per token in pages.
    Layers with equal needs share a group (one page pool, one block table per
    request).  `window` keys at most are ever read again; None means all."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class FixedState:
    """Cache need of a mixer that keeps a state of fixed size per request: one
    slot of `shape` float32 values, zeroed when the request is created."""

    shape: tuple[int, ...]


CacheNeed = PagedKeyValue | FixedState | None


class Part:
    """Base of norms, position encodings, mixers, feed-forwards and blocks."""

    kind: ClassVar[str] = ""
    # Whether a step through the part is the same sequence of kernel launches whatever the data:
    # then a step of single tokens may be captured into a graph once and replayed.  A part that
    # looks at values on the host (routing that gathers rows, a loop over a request's tokens) says False.
    replayable: ClassVar[bool] = True

    @classmethod
    def tensors(cls, spec: Any) -> dict[str, TensorSpec]:
        """Names (relative to the part's prefix) and shapes of its tensors."""
        return {}

    @classmethod
    def cache_need(cls, spec: Any) -> CacheNeed:
        return None

    def __init__(self, spec: Any, tensors: dict[str, torch.Tensor], kernels: Any) -> None:
        self.spec = spec
        self.kernels = kernels


class Registry:
    """kind -> part class, for one family of parts."""

    def __init__(self, family: str) -> None:
        self.family = family
        self._classes: dict[str, type[Part]] = {}

    def register(self, kind: str):
        def decorate(cls: type[Part]) -> type[Part]:
            if kind in self._classes and self._classes[kind] is not cls:
                raise ValueError(f"{self.family} kind {kind!r} is already registered")
            cls.kind = kind
            self._classes[kind] = cls
            return cls

        return decorate

    def unregister(self, kind: str) -> None:
        self._classes.pop(kind, None)

    def get(self, spec: Any) -> type[Part]:
        kind = getattr(spec, "kind", None)
        if kind not in self._classes:
            known = ", ".join(sorted(self._classes)) or "none"
            raise KeyError(f"no {self.family} of kind {kind!r} is registered (known: {known})")
        return self._classes[kind]

    def tensors(self, spec: Any) -> dict[str, TensorSpec]:
        return self.get(spec).tensors(spec)

    def cache_need(self, spec: Any) -> CacheNeed:
        return self.get(spec).cache_need(spec)

    def build(self, spec: Any, tensors: dict[str, torch.Tensor], kernels: Any) -> Part:
        return self.get(spec)(spec, tensors, kernels)

    def kinds(self) -> list[str]:
        return sorted(self._classes)


NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")
# What acts on the residual stream between the embedding and the first layer (`forward(hidden, batch)`, in
# place: a table of absolute positions, a scale), and on the logits after the head (`forward(logits, batch)
# -> logits`: a bias, a soft cap).  Qwen2 has neither; a model lists them in `ModelSpec.input_parts` and
# `ModelSpec.output_parts`.
STREAM_PARTS = Registry("part on the embedded stream")
LOGIT_PARTS = Registry("part on the logits")


def under(tensors: dict[str, Any], prefix: str) -> dict[str, Any]:
    """The entries of `tensors` below `prefix`, with the prefix removed."""
    return {name[len(prefix):]: value for name, value in tensors.items() if name.startswith(prefix)}


def prefixed(tensors: dict[str, Any], prefix: str) -> dict[str, Any]:
    return {prefix + name: value for name, value in tensors.items()}
