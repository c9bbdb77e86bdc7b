"""Which kernel libraries exist, and with which compile-time constants the
repository's own tests, smoke run and benchmark need them."""

from __future__ import annotations

# module -> list of constant sets
DEFAULT_VARIANTS: dict[str, list[dict[str, object]]] = {
    "elementwise": [{}],
    "gemm_generic": [{}],
    "gemm_bf16": [{}],
    "attention_generic": [{}],
    "sampling": [{}],
}
