"""Reads a model folder (config.json + *.safetensors) into tensors by name.

Like the reference's loader (`src/llmserve/checkpoint.py:28-70`) it walks every
safetensors file in sorted order and matches tensors by their name in the file,
without renaming, transposing or splitting.  Unlike it, nothing is skipped in
silence: tensors the model does not know, tensors it misses and wrong shapes
are all collected and reported in one error.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any

import torch

from ..config.model import ArchitectureConfig
from ..parts.base import TensorSpec
from ..parts.model import ModelSpec
from ..registry import Architecture, resolve_architecture


class WeightsError(ValueError):
    """The tensors of a model folder do not fit the model.  Lists everything wrong."""

    def __init__(self, where: str, missing, unexpected, wrong_shapes, wrong_types=()) -> None:
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shapes = sorted(wrong_shapes)
        self.wrong_types = sorted(wrong_types)
        lines = [f"weights in {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shapes:
            lines.append(f"  wrong shape: {name} is {list(got)}, the model needs {list(want)}")
        for name, got, want in self.wrong_types:
            lines.append(f"  wrong type: {name} is {got}, the model needs {want}")
        super().__init__("\n".join(lines))


@dataclass
class LoadedModel:
    architecture: Architecture
    config: ArchitectureConfig
    spec: ModelSpec
    tensors: dict[str, torch.Tensor]
    dtype: torch.dtype


RUN_DTYPES = {
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
    "float32": torch.float32,
    "fp32": torch.float32,
    torch.bfloat16: torch.bfloat16,
    torch.float32: torch.float32,
}

_WIDE = (torch.float32, torch.float64)


def run_dtype(name: Any) -> torch.dtype:
    if name not in RUN_DTYPES:
        raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}")
    return RUN_DTYPES[name]


def read_config(folder: str | Path) -> tuple[Architecture, ArchitectureConfig]:
    """The architecture and typed configuration of a model folder, or of a config.json given by its path."""
    path = Path(folder)
    if path.is_dir():
        path = path / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json under {folder}")
    values = json.loads(path.read_text())
    architecture = resolve_architecture(values)
    return architecture, architecture.config_class.from_dict(values)


def _kept_as(tensor: torch.Tensor, spec: TensorSpec, dtype: torch.dtype) -> torch.Tensor:
    """Integer tables as int32; a tensor stored in 32 bits (or more) stays float32;
    everything else in the run dtype."""
    if spec.integer:
        return tensor.to(torch.int32)
    if dtype == torch.float32 or tensor.dtype in _WIDE:
        return tensor.to(torch.float32)
    return tensor.to(dtype)


def fit_tensors(
    expected: dict[str, TensorSpec],
    found: dict[str, Any],
    where: str,
    optional: set[str] = frozenset(),
) -> None:
    """Raises one `WeightsError` for everything that does not fit.  `found`
    maps names to objects with `.shape` and `.dtype`."""
    missing = [name for name in expected if name not in found and name not in optional]
    unexpected = [name for name in found if name not in expected]
    wrong_shapes, wrong_types = [], []
    for name, spec in expected.items():
        if name not in found:
            continue
        shape = tuple(found[name].shape)
        if shape != tuple(spec.shape):
            wrong_shapes.append((name, shape, tuple(spec.shape)))
        floating = found[name].dtype.is_floating_point
        if floating == spec.integer:
            want = "integer" if spec.integer else "floating point"
            wrong_types.append((name, str(found[name].dtype), want))
    if missing or unexpected or wrong_shapes or wrong_types:
        raise WeightsError(where, missing, unexpected, wrong_shapes, wrong_types)


def load_model_folder(
    folder: str | Path, dtype: Any = "bfloat16", device: str | torch.device = "cpu"
) -> LoadedModel:
    """config.json chooses the architecture; tensors are matched by name.  A
    name may carry the `model.` prefix or not (`checkpoint.py:52`)."""
    from safetensors import safe_open

    folder = Path(folder)
    dtype = run_dtype(dtype)
    architecture, config = read_config(folder)
    spec = architecture.build_spec(config)
    expected = spec.tensors()
    files = sorted(folder.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no safetensors files under {folder}")  # `checkpoint.py:47-48`

    def model_name(name: str) -> str:
        if name in expected:
            return name
        for candidate in ("model." + name, name.removeprefix("model.")):
            if candidate in expected:
                return candidate
        return name

    found: dict[str, torch.Tensor] = {}
    for path in files:
        with safe_open(str(path), framework="pt", device="cpu") as source:
            for source_name in source.keys():
                found[source_name] = source.get_tensor(source_name)
    if architecture.adapt_tensors is not None:  # the files name or cut their tensors otherwise than the parts do
        found = architecture.adapt_tensors(found, config)
    found = {model_name(name): tensor for name, tensor in found.items()}

    # A tied model's file may still carry the head: fine if it is the embedding.
    if spec.tie_embeddings and spec.head_name in found:
        embedding = found.get(spec.embedding_name)
        if embedding is not None and embedding.shape == found[spec.head_name].shape and torch.equal(
            embedding, found[spec.head_name]
        ):
            del found[spec.head_name]
    fit_tensors(expected, found, str(folder))
    tensors = {
        name: _kept_as(found[name], expected[name], dtype).to(device).contiguous() for name in expected
    }
    return LoadedModel(architecture, config, spec, tensors, dtype)
