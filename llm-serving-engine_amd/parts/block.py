"""How a layer's parts are arranged."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, CacheNeed, Part, TensorSpec, prefixed, under


class Block(Part):
    """`forward(hidden, delta, batch, cell)`: `hidden` is the float32 residual
    stream [T, hidden] and `delta` what the layer before still has to add to it
    (None at the first layer).  Returns this layer's own pending delta."""

    def forward(self, hidden, delta, batch, cell) -> torch.Tensor:
        raise NotImplementedError


@dataclass(frozen=True)
class PreNormBlockSpec:
    """h += mixer(norm(h)); h += feed_forward(norm(h)).  The `*_name` fields are
    the prefixes of the sub-parts' tensors below the layer's own prefix."""

    mixer_norm: Any
    mixer: Any
    feed_forward_norm: Any
    feed_forward: Any
    mixer_norm_name: str = "input_layernorm."
    mixer_name: str = "self_attn."
    feed_forward_norm_name: str = "post_attention_layernorm."
    feed_forward_name: str = "mlp."
    kind: str = "prenorm"


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    """Reference `model.py:199-201`.  Each residual add is done by the norm that
    follows it, so the stream is read and written once per sub-layer."""

    @classmethod
    def _members(cls, spec: PreNormBlockSpec):
        return (
            (spec.mixer_norm_name, NORMS, spec.mixer_norm),
            (spec.mixer_name, MIXERS, spec.mixer),
            (spec.feed_forward_norm_name, NORMS, spec.feed_forward_norm),
            (spec.feed_forward_name, FEED_FORWARDS, spec.feed_forward),
        )

    @classmethod
    def tensors(cls, spec: PreNormBlockSpec) -> dict[str, TensorSpec]:
        found: dict[str, TensorSpec] = {}
        for name, registry, member in cls._members(spec):
            found.update(prefixed(registry.tensors(member), name))
        return found

    @classmethod
    def cache_need(cls, spec: PreNormBlockSpec) -> CacheNeed:
        return MIXERS.cache_need(spec.mixer)

    def __init__(self, spec: PreNormBlockSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        built = [
            registry.build(member, under(tensors, name), kernels)
            for name, registry, member in self._members(spec)
        ]
        self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward = built
        self.replayable = all(part.replayable for part in built)

    def forward(self, hidden, delta, batch, cell) -> torch.Tensor:
        normed = self.mixer_norm.forward(hidden, delta)
        mixed = self.mixer.forward(normed, batch, cell)
        normed = self.feed_forward_norm.forward(hidden, mixed)
        return self.feed_forward.forward(normed, batch)
