"""Position encodings that act on queries and keys before they are cached."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import POSITIONS, Part


@dataclass(frozen=True)
class HeadLayout:
    """How one token's projected row is laid out: q heads, then k heads, then v heads."""

    num_heads: int
    num_kv_heads: int
    head_dim: int

    @property
    def width(self) -> int:
        return (self.num_heads + 2 * self.num_kv_heads) * self.head_dim


@dataclass(frozen=True)
class RotarySpec:
    head_dim: int
    theta: float
    pairing: str = "half"  # "half": (j, j + D/2); "adjacent": (2j, 2j+1)
    kind: str = "rotary"


@dataclass(frozen=True)
class NoPositionSpec:
    kind: str = "none"


class PositionEncoding(Part):
    def encode_and_store(self, qkv, layout: HeadLayout, batch, cell) -> None:
        """Encodes q and k of `qkv` [T, layout.width] in place by each token's
        position and, if `cell` is writable, stores k and v in the cell's pages."""
        raise NotImplementedError

    def encode_store_attend(self, qkv, layout: HeadLayout, batch, cell, scale: float, window, project=None) -> "torch.Tensor":
        """`encode_and_store`, then attention over the cell's pages; with `project` (a prepared linear),
        then that product of the result, in float32, possibly as partial sums.  An encoding that a kernel
        can apply on the way (rotary) overrides this to let the kernel library fuse what it can."""
        self.encode_and_store(qkv, layout, batch, cell)
        mixed = self.kernels.paged_attention(qkv, layout, batch, cell, scale, window)
        if project is None:
            return mixed
        return self.kernels.linear(mixed, project, out_dtype=torch.float32, partial=True)


@POSITIONS.register("rotary")
class Rotary(PositionEncoding):
    """Reference `model.py:26-43`: inv[j] = theta^(-2j/D), angle = position *
    inv[j] in float32; the pair (a, b) becomes (a cos - b sin, b cos + a sin).
    The reference gathers cos/sin from a table built at start-up; here the
    kernel computes them from the position, in float32, so no length is fixed."""

    def __init__(self, spec: RotarySpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if spec.pairing not in ("half", "adjacent"):
            raise ValueError(f"unknown rotary pairing {spec.pairing!r}")
        # one tensor per (head size, theta) and kernel library: layers that rotate alike share it,
        # and with it whatever the library derives from it per step
        shared = kernels.__dict__.setdefault("_rotary_frequencies", {})
        key = (spec.head_dim, spec.theta)
        if key not in shared:
            exponents = torch.arange(0, spec.head_dim, 2, dtype=torch.float32) / spec.head_dim
            shared[key] = kernels.to_device(1.0 / (spec.theta ** exponents))
        self.inverse_frequencies = shared[key]

    def encode_and_store(self, qkv, layout: HeadLayout, batch, cell) -> None:
        self.kernels.rotate_and_store(
            qkv, layout, batch, cell, self.inverse_frequencies, self.spec.pairing
        )

    def encode_store_attend(self, qkv, layout: HeadLayout, batch, cell, scale: float, window, project=None):
        return self.kernels.rotate_store_attend(
            qkv, layout, batch, cell, self.inverse_frequencies, self.spec.pairing, scale, window, project=project
        )


@POSITIONS.register("none")
class NoPosition(PositionEncoding):
    """No encoding: keys and values are only stored."""

    def encode_and_store(self, qkv, layout: HeadLayout, batch, cell) -> None:
        self.kernels.rotate_and_store(qkv, layout, batch, cell, None, "none")

    def encode_store_attend(self, qkv, layout: HeadLayout, batch, cell, scale: float, window, project=None):
        return self.kernels.rotate_store_attend(qkv, layout, batch, cell, None, "none", scale, window, project=project)
