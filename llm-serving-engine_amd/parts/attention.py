"""The attention mixer: projections, position encoding, paged attention."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from .base import MIXERS, POSITIONS, PagedKeyValue, Part, TensorSpec
from .position import HeadLayout


class Mixer(Part):
    """A token mixer.  `forward(x, batch, cell)` takes the normed rows [T, hidden]
    in the run dtype and returns the float32 rows [T, hidden] to add to the
    residual stream, or partial sums [parts, T, hidden] of them (whoever adds
    them to the stream adds the parts in order).  `cell` is what `cache_need`
    asked for."""

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        raise NotImplementedError


@dataclass(frozen=True)
class AttentionSpec:
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    position: Any  # spec of a position encoding
    qkv_bias: bool = True
    out_bias: bool = False
    window: int | None = None
    kind: str = "attention"


@MIXERS.register("attention")
class Attention(Mixer):
    """Grouped-query attention over the paged cache (reference `model.py:46-177`).

    q = x Wq^T + bq, k, v likewise; position encoding on q and k; k and v of
    every token of the step are stored before any row attends (`:114-121`);
    query head h reads kv head h // G (`:84-86`); softmax(q.k * scale) over the
    keys at positions (p - window, p]; output projection (`:66`).  The three
    projections run as one product over the concatenated weight.
    """

    @classmethod
    def tensors(cls, spec: AttentionSpec) -> dict[str, TensorSpec]:
        q_size = spec.num_heads * spec.head_dim
        kv_size = spec.num_kv_heads * spec.head_dim
        found = {
            "q_proj.weight": TensorSpec((q_size, spec.hidden_size)),
            "k_proj.weight": TensorSpec((kv_size, spec.hidden_size)),
            "v_proj.weight": TensorSpec((kv_size, spec.hidden_size)),
            "o_proj.weight": TensorSpec((spec.hidden_size, q_size)),
        }
        if spec.qkv_bias:
            found["q_proj.bias"] = TensorSpec((q_size,), role="bias")
            found["k_proj.bias"] = TensorSpec((kv_size,), role="bias")
            found["v_proj.bias"] = TensorSpec((kv_size,), role="bias")
        if spec.out_bias:
            found["o_proj.bias"] = TensorSpec((spec.hidden_size,), role="bias")
        # a position encoding with tensors of its own (a learned table) keeps them below "position."
        for name, tensor in POSITIONS.tensors(spec.position).items():
            found["position." + name] = tensor
        return found

    @classmethod
    def cache_need(cls, spec: AttentionSpec) -> PagedKeyValue:
        return PagedKeyValue(spec.num_kv_heads, spec.head_dim, spec.window)

    def __init__(self, spec: AttentionSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.layout = HeadLayout(spec.num_heads, spec.num_kv_heads, spec.head_dim)
        names = ("q_proj", "k_proj", "v_proj")
        bias = [tensors[f"{name}.bias"] for name in names] if spec.qkv_bias else None
        self.qkv = kernels.prepare_linear([tensors[f"{name}.weight"] for name in names], bias)
        self.out = kernels.prepare_linear(
            [tensors["o_proj.weight"]], [tensors["o_proj.bias"]] if spec.out_bias else None
        )
        own = {name[len("position."):]: tensor for name, tensor in tensors.items() if name.startswith("position.")}
        self.position = POSITIONS.build(spec.position, own, kernels)
        self.replayable = self.position.replayable

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        qkv = self.kernels.linear(x, self.qkv)
        # the output projection goes with the attention: a kernel library may fuse the two (key splits of
        # a decode step merged by the product that reads them)
        return self.position.encode_store_attend(
            qkv, self.layout, batch, cell, self.spec.scale, self.spec.window, project=self.out
        )
