"""Random weights from a configuration and a seed, written as a model folder.

The reference draws every Linear/Embedding weight from N(0, 0.02), zeroes the
biases and sets norm weights to one, in module construction order under one
global seed (`model.py:251-258`, `cli.py:40-41`).  Here each tensor is drawn
from its own generator seeded by (seed, tensor name), so the values do not
depend on the order of construction, and biases and norm weights can be drawn
too (zero biases and unit norms hide faults).
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Any

import torch

from ..config.model import ArchitectureConfig
from ..parts.base import TensorSpec
from ..parts.model import ModelSpec
from ..registry import ARCHITECTURES


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(
    name: str,
    spec: TensorSpec,
    seed: int,
    *,
    std: float = 0.02,
    bias_std: float = 0.02,
    norm_std: float = 0.0,
    device: str | torch.device = "cpu",
) -> torch.Tensor:
    """One float32 (or int32) tensor; the same (seed, name) gives the same values on one device type."""
    generator = torch.Generator(device=device).manual_seed(_seed_for(seed, name))
    if spec.integer:
        return torch.randint(0, 1 << 15, spec.shape, generator=generator, device=device, dtype=torch.int32)
    if spec.role == "norm":
        if norm_std == 0.0:
            return torch.ones(spec.shape, device=device)
        return 1.0 + norm_std * torch.randn(spec.shape, generator=generator, device=device)
    scale = bias_std if spec.role == "bias" else std
    return scale * torch.randn(spec.shape, generator=generator, device=device)


def random_tensors(
    spec: ModelSpec,
    seed: int,
    *,
    dtype: torch.dtype = torch.bfloat16,
    wide_roles: tuple[str, ...] = (),
    device: str | torch.device = "cpu",
    **scales: float,
) -> dict[str, torch.Tensor]:
    """Every tensor of the model, in `dtype` except roles in `wide_roles`, which stay float32."""
    tensors = {}
    for name, tensor_spec in spec.tensors().items():
        value = random_tensor(name, tensor_spec, seed, device=device, **scales)
        if not tensor_spec.integer and tensor_spec.role not in wide_roles:
            value = value.to(dtype)
        tensors[name] = value
    return tensors


def random_model(
    config: ArchitectureConfig | dict | str | Path,
    seed: int,
    *,
    dtype: Any = torch.bfloat16,
    device: str | torch.device = "cpu",
    **scales: float,
):
    """A model with seeded random weights made in memory, on `device`: `config` is a typed
    configuration, the mapping of a config.json, or the path of one (its architecture is
    resolved as for a model folder).  Large configurations need no folder on disk this way."""
    from ..registry import resolve_architecture
    from .loader import LoadedModel, run_dtype

    if isinstance(config, (str, Path)):
        config = json.loads(Path(config).read_text())
    if isinstance(config, dict):
        architecture = resolve_architecture(config)
        config = architecture.config_class.from_dict(config)
    else:
        architecture = ARCHITECTURES[config.architecture]
    dtype = run_dtype(dtype)
    spec = architecture.build_spec(config)
    tensors = random_tensors(spec, seed, dtype=dtype, device=device, **scales)
    return LoadedModel(architecture, config, spec, tensors, dtype)


def write_model_folder(
    folder: str | Path,
    config: ArchitectureConfig,
    seed: int,
    *,
    dtype: torch.dtype = torch.bfloat16,
    wide_roles: tuple[str, ...] = (),
    extra_config: dict[str, Any] | None = None,
    **scales: float,
) -> Path:
    """Writes config.json and model.safetensors for `config` and returns the folder."""
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    architecture = ARCHITECTURES[config.architecture]
    spec = architecture.build_spec(config)
    tensors = random_tensors(spec, seed, dtype=dtype, wide_roles=wide_roles, **scales)
    values = config.to_config_json()
    values.update(extra_config or {})
    (folder / "config.json").write_text(json.dumps(values, indent=2) + "\n")
    save_file({name: value.contiguous() for name, value in tensors.items()}, str(folder / "model.safetensors"))
    return folder
