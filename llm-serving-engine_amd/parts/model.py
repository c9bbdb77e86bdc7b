"""A decoder as data: an embedding, layer definitions, the order in which they
run, a final norm and an output head.  `DecoderModel` runs any such list."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from .base import BLOCKS, LOGIT_PARTS, NORMS, STREAM_PARTS, CacheNeed, TensorSpec, prefixed, under


@dataclass(frozen=True)
class LayerDefinition:
    prefix: str  # e.g. "model.layers.3."
    block: Any  # spec of a block


@dataclass(frozen=True)
class LayerRun:
    """One entry of the run order.  `layer` indexes `ModelSpec.layers`; a layer
    may be named by several entries (its tensors are shared, each run has a
    cache cell of its own).  With `reads` set, the run uses the cell of that
    earlier entry of the run order instead, and stores nothing."""

    layer: int
    reads: int | None = None


@dataclass(frozen=True)
class NamedPart:
    """A part outside the layers: the prefix of its tensors and its spec."""

    prefix: str
    spec: Any


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    layers: tuple[LayerDefinition, ...]
    run_order: tuple[LayerRun, ...]
    final_norm: Any
    tie_embeddings: bool
    embedding_name: str = "model.embed_tokens.weight"
    final_norm_name: str = "model.norm."
    head_name: str = "lm_head.weight"
    # parts that act on the embedded rows before the first layer (kinds of STREAM_PARTS), and on the
    # logits after the head (kinds of LOGIT_PARTS), in order; Qwen2 has none
    input_parts: tuple[NamedPart, ...] = ()
    output_parts: tuple[NamedPart, ...] = ()

    def __post_init__(self) -> None:
        for index, run in enumerate(self.run_order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"run {index} names layer {run.layer}, which does not exist")
            if run.reads is not None:
                if not 0 <= run.reads < index:
                    raise ValueError(f"run {index} reads the cache of run {run.reads}, which is not earlier")
                if self.run_order[run.reads].reads is not None:
                    raise ValueError(f"run {index} reads run {run.reads}, which owns no cache")
                if self.cell_need(run.reads) != self.cell_need(index):
                    raise ValueError(f"run {index} and run {run.reads} need different caches")

    def cell_need(self, run_index: int) -> CacheNeed:
        block = self.layers[self.run_order[run_index].layer].block
        return BLOCKS.cache_need(block)

    def tensors(self) -> dict[str, TensorSpec]:
        """Every tensor of the model by its name in the model folder."""
        found = {self.embedding_name: TensorSpec((self.vocab_size, self.hidden_size), role="embedding")}
        for layer in self.layers:
            found.update(prefixed(BLOCKS.tensors(layer.block), layer.prefix))
        found.update(prefixed(NORMS.tensors(self.final_norm), self.final_norm_name))
        for part in self.input_parts:
            found.update(prefixed(STREAM_PARTS.tensors(part.spec), part.prefix))
        for part in self.output_parts:
            found.update(prefixed(LOGIT_PARTS.tensors(part.spec), part.prefix))
        if not self.tie_embeddings:
            found[self.head_name] = TensorSpec((self.vocab_size, self.hidden_size))
        return found


class DecoderModel:
    """Runs a `ModelSpec`: embedding, the layers in run order, final norm and
    head on the wanted rows only (the reference computes the head on every row,
    `model.py:309`).  Architecture-agnostic: everything specific sits in the spec."""

    def __init__(self, spec: ModelSpec, tensors: dict[str, torch.Tensor], kernels) -> None:
        self.spec = spec
        self.kernels = kernels
        self.embedding = tensors[spec.embedding_name]
        self.layers = [
            BLOCKS.build(layer.block, under(tensors, layer.prefix), kernels) for layer in spec.layers
        ]
        self.final_norm = NORMS.build(spec.final_norm, under(tensors, spec.final_norm_name), kernels)
        head = self.embedding if spec.tie_embeddings else tensors[spec.head_name]
        self.head = kernels.prepare_linear([head], None)
        self.input_parts = [STREAM_PARTS.build(part.spec, under(tensors, part.prefix), kernels) for part in spec.input_parts]
        self.output_parts = [LOGIT_PARTS.build(part.spec, under(tensors, part.prefix), kernels) for part in spec.output_parts]
        every = [*self.layers, self.final_norm, *self.input_parts, *self.output_parts]
        self.replayable = all(part.replayable for part in every)

    def _run_layers(self, batch, cells: list):
        hidden = self.kernels.embedding(self.embedding, batch.token_ids)
        for part in self.input_parts:
            part.forward(hidden, batch)
        delta = None
        for run, cell in zip(self.spec.run_order, cells):
            delta = self.layers[run.layer].forward(hidden, delta, batch, cell)
        return hidden, delta

    def forward_without_logits(self, batch, cells: list) -> None:
        """Runs the layers only: the step fills the cache and no logits are wanted."""
        self._run_layers(batch, cells)

    def forward(self, batch, cells: list) -> torch.Tensor:
        """Logits [R, vocab] float32 at `batch.logit_rows`.  `cells[i]` is the
        cache cell of run i."""
        hidden, delta = self._run_layers(batch, cells)
        if getattr(batch, "every_row_wanted", False):  # the final norm adds the last layer's delta itself
            normed = self.final_norm.forward(hidden, delta)
        else:
            rows = self.kernels.gather_rows(hidden, delta, batch.logit_rows)
            normed = self.final_norm.forward(rows, None)
        logits = self.kernels.linear(normed, self.head, out_dtype=torch.float32)
        for part in self.output_parts:
            logits = part.forward(logits, batch)
        return logits
