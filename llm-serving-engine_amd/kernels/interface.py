"""The operations the parts call.  The product has one implementation, the HIP
library in `hip.py`; the interface is spelled out so that tests can check parts,
cache and step function with a stand-in of their own on a machine without a GPU.

Conventions: the residual stream and every value added to it are float32 in
every run dtype; activations between kernels are in the run dtype (bfloat16 or
float32); products accumulate in float32; logits are float32.
"""

from __future__ import annotations

from typing import Any, Protocol

import torch


class Kernels(Protocol):
    device: torch.device
    dtype: torch.dtype

    def to_device(self, tensor: torch.Tensor) -> torch.Tensor: ...

    def queued_to_device(self, tensor: torch.Tensor) -> torch.Tensor:
        """As `to_device`, for small per-step inputs: the host does not wait for work queued before."""

    def embedding(self, table: torch.Tensor, token_ids: torch.Tensor) -> torch.Tensor:
        """float32 rows [T, hidden] of `table` at `token_ids`."""

    def add_rms_norm(
        self, hidden: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float
    ) -> torch.Tensor:
        """`hidden += delta` in place (float32), then rows * rsqrt(mean(rows^2) + eps) * weight in the run dtype."""

    def prepare_linear(self, weights: list[torch.Tensor], biases: list[torch.Tensor] | None) -> Any:
        """Concatenates [N_i, K] weights (and biases) along N into whatever layout `linear` wants."""

    def prepare_gated_linear(self, gate: torch.Tensor, up: torch.Tensor, activation: str = "silu") -> Any:
        """Gate and up weights [I, K] in whatever layout `gated_linear` wants; `activation` is the gate's
        (silu, gelu, gelu_tanh, relu), and one the library has no kernel for is refused here, by name."""

    def linear(
        self, x: torch.Tensor, weights: Any, out_dtype: torch.dtype | None = None, *, partial: bool = False
    ) -> torch.Tensor:
        """x [T, K] @ W^T + bias -> [T, N] in `out_dtype` (the run dtype if None).  With
        `partial`, a float32 result may be [parts, T, N] partial sums for the reader to add."""

    def gated_linear(self, x: torch.Tensor, weights: Any) -> torch.Tensor:
        """act(x Wg^T) * (x Wu^T) -> [T, I] in the run dtype."""

    def rotate_and_store(
        self, qkv: torch.Tensor, layout: Any, batch: Any, cell: Any,
        inverse_frequencies: torch.Tensor | None, pairing: str,
    ) -> None:
        """Rotary on the q and k heads of `qkv` in place; k and v into the cell's pages if it is writable."""

    def paged_attention(
        self, qkv: torch.Tensor, layout: Any, batch: Any, cell: Any, scale: float, window: int | None, *,
        score_slopes: torch.Tensor | None = None, soft_cap: float | None = None,
    ) -> torch.Tensor:
        """Attention of the q heads of `qkv` over the cell's pages -> [T, heads * head_dim].
        Before the softmax a score s of a query at position p for a key at position k may be changed,
        for encodings and models that want it (Qwen2 wants neither): with `soft_cap`, to
        soft_cap * tanh(s / soft_cap); with `score_slopes` (float32, one per query head), by
        - slope * (p - k) after that.  A library refuses what it cannot compute."""

    def rotate_store_attend(
        self, qkv: torch.Tensor, layout: Any, batch: Any, cell: Any,
        inverse_frequencies: torch.Tensor | None, pairing: str, scale: float, window: int | None,
        project: Any = None,
    ) -> torch.Tensor:
        """`rotate_and_store` followed by `paged_attention` (a library may fuse them); with `project` (what
        `prepare_linear` returned), followed by `linear(that, project, float32, partial=True)`, whose result
        is returned instead (a library may let that product finish what the attention left undone)."""

    def gather_rows(self, hidden: torch.Tensor, delta: torch.Tensor | None, rows: torch.Tensor) -> torch.Tensor:
        """float32 (hidden + delta)[rows]."""

    def argmax(self, logits: torch.Tensor) -> torch.Tensor: ...

    def sample(
        self, logits: torch.Tensor, temperatures: torch.Tensor, top_ps: torch.Tensor, uniforms: torch.Tensor,
        with_top_p: bool = True,
    ) -> torch.Tensor:
        """One token per row.  `with_top_p=False` promises that no row with a temperature has top_p < 1
        (a library may then leave the search for the kept set out)."""
