"""Which kernel libraries exist, and with which compile-time constants the
repository's own tests, smoke run and benchmark need them."""

from __future__ import annotations

# module -> list of constant sets
DEFAULT_VARIANTS: dict[str, list[dict[str, object]]] = {
    "elementwise": [{}],
    "gemm_generic": [{}],
    "gemm_f32": [{}],
    "gemm_bf16": [{}],
    "attention_generic": [{}],
    "sampling": [{}],
    # head sizes of the tests' models and kernel tests, and of the benchmark
    "attention_bf16": [{"HEAD_DIM": d} for d in (16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256)],
    "attention_f32": [{"HEAD_DIM": d} for d in (16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256)],
}
