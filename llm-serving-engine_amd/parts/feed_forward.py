"""Feed-forward parts."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import FEED_FORWARDS, Part, TensorSpec


class FeedForward(Part):
    """`forward(x)` takes the normed rows [T, hidden] in the run dtype and
    returns the float32 rows to add to the residual stream, or partial sums
    [parts, T, hidden] of them."""

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


@dataclass(frozen=True)
class GatedMLPSpec:
    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    kind: str = "gated_mlp"


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(FeedForward):
    """down(act(gate(x)) * up(x)) without biases (reference `model.py:180-188`).
    Gate and up run as one product whose epilogue applies act(gate) * up."""

    @classmethod
    def tensors(cls, spec: GatedMLPSpec) -> dict[str, TensorSpec]:
        return {
            "gate_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
            "up_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
            "down_proj.weight": TensorSpec((spec.hidden_size, spec.intermediate_size)),
        }

    def __init__(self, spec: GatedMLPSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        # the kernel library says which activations it has, and refuses another by name
        self.gate_up = kernels.prepare_gated_linear(
            tensors["gate_proj.weight"], tensors["up_proj.weight"], spec.activation
        )
        self.down = kernels.prepare_linear([tensors["down_proj.weight"]], None)

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        activated = self.kernels.gated_linear(x, self.gate_up)
        return self.kernels.linear(activated, self.down, out_dtype=torch.float32, partial=True)
