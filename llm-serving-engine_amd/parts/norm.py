"""Normalisation parts."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import NORMS, Part, TensorSpec


@dataclass(frozen=True)
class RMSNormSpec:
    size: int
    eps: float
    kind: str = "rmsnorm"


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    """y = x * rsqrt(mean(x^2) + eps) * weight (reference `model.py:14-23`), with
    the residual add in front of it: `hidden += delta` happens in the same
    kernel, in float32, and `hidden` stays float32 in every run dtype."""

    @classmethod
    def tensors(cls, spec: RMSNormSpec) -> dict[str, TensorSpec]:
        return {"weight": TensorSpec((spec.size,), role="norm")}

    def __init__(self, spec: RMSNormSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.weight = tensors["weight"]

    def forward(self, hidden: torch.Tensor, delta: torch.Tensor | None) -> torch.Tensor:
        """Adds `delta` into `hidden` (in place) and returns the normed rows in the run dtype."""
        return self.kernels.add_rms_norm(hidden, delta, self.weight, self.spec.eps)
