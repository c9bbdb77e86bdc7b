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


KEY_PIECE = 8  # elements of a key that stay together in a page (csrc/common.h has the same number)


def key_piece_width(head_dim: int) -> int:
    """A key is kept in pieces of KEY_PIECE elements; a head size that is no multiple of it in one piece."""
    return KEY_PIECE if head_dim % KEY_PIECE == 0 else head_dim


VALUE_PIECE = 8  # keys whose values of one dimension stay together in a page (csrc/common.h has the same number)


def value_piece_width(page_size: int) -> int:
    """A page's values are kept in pieces of VALUE_PIECE keys; a page size that is no multiple of it in one piece."""
    return VALUE_PIECE if page_size % VALUE_PIECE == 0 else page_size


class CacheNeed:
    """What a part keeps in the cache from one step to the next.  The cache manager knows two ways of
    giving room, and a need is of one of them: `PagedNeed` (an entry per token, in pages that a request
    holds through a block table) or `SlotNeed` (one entry of fixed size per request).  What an entry *is*
    is the need's own business: a new kind of need is a subclass that says what a page of it holds, and
    nothing in the cache manager, the step function or the scheduler changes.  Needs are compared and
    hashed (frozen dataclasses): runs with equal paged needs share a pool and a block table per request."""


class PagedNeed(CacheNeed):
    """An entry per token.  A subclass has a field `window` (keys at most that are ever read again, None:
    all) and says what one page holds."""

    window: int | None = None

    def page_fields(self, page_size: int) -> dict[str, tuple[int, ...]]:
        """name -> shape of ONE page of that field.  The cache keeps each field as a tensor
        [pages, *shape] in the run dtype, and a `CacheCell` shows them by these names."""
        raise NotImplementedError

    def token_rows(self, page: dict[str, torch.Tensor], page_size: int) -> dict[str, torch.Tensor]:
        """One page's fields rearranged so that the token's offset in the page leads: name ->
        [page_size, ...].  The host-side read path (tests, debugging) walks pages through it; kernels
        read the pages as they lie."""
        raise NotImplementedError


class SlotNeed(CacheNeed):
    """One entry of fixed size per request.  A subclass has a field `shape`: the cache keeps a float32
    tensor [request slots, *shape], zeroed when a request takes its slot."""

    shape: tuple[int, ...] = ()


@dataclass(frozen=True)
class PagedKeyValue(PagedNeed):
    """Cache need of a mixer that keeps a key and a value per token in pages.  Keys lie in pieces of
    eight elements, the same piece of all the keys of a page side by side ([kv_heads, head_dim / w,
    page_size, w], w = `key_piece_width(head_dim)`): the matrix cores take keys as rows, a lane holding
    one piece of one key and its neighbours that piece of the next keys, and neighbouring lanes should
    read neighbouring bytes.  Values are stored transposed, in pieces of eight keys ([kv_heads, page_size / v,
    head_dim, v], v = `value_piece_width(page_size)`): attention sums over keys, the matrix cores want the
    summed index contiguous, and a lane's neighbours hold the same keys of the next dimensions."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None

    def page_fields(self, page_size: int) -> dict[str, tuple[int, ...]]:
        width = key_piece_width(self.head_dim)
        return {
            "keys": (self.num_kv_heads, self.head_dim // width, page_size, width),
            "values": (self.num_kv_heads, page_size // value_piece_width(page_size), self.head_dim, value_piece_width(page_size)),
        }

    def token_rows(self, page: dict[str, torch.Tensor], page_size: int) -> dict[str, torch.Tensor]:
        keys = page["keys"].permute(2, 0, 1, 3).reshape(page_size, self.num_kv_heads, self.head_dim)
        values = page["values"].permute(1, 3, 0, 2).reshape(page_size, self.num_kv_heads, self.head_dim)
        return {"keys": keys, "values": values}


@dataclass(frozen=True)
class FixedState(SlotNeed):
    """Cache need of a mixer that keeps a state of fixed size per request: one
    slot of `shape` float32 values, zeroed when the request is created."""

    shape: tuple[int, ...]


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
    def cache_need(cls, spec: Any) -> "CacheNeed | dict[str, CacheNeed] | None":
        """What the part keeps in the cache: nothing, one need, or several by name (a block with two
        mixers side by side, one with pages and one with a state): its cell is then a dict of cells
        by the same names."""
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

    def cache_need(self, spec: Any) -> "CacheNeed | dict[str, CacheNeed] | None":
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
