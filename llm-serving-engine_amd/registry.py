"""One registry from an architecture's name to its model.

An architecture is a typed configuration class plus a function that turns a
configuration into a `ModelSpec`; the generic `DecoderModel` runs the spec.
The reference has no registry: it accepts config.json only when `model_type`
is "qwen2" (`checkpoint.py:34-36`) and always builds its one `Transformer`.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

from .config.model import ArchitectureConfig, ConfigError
from .parts.model import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type[ArchitectureConfig]
    build_spec: Callable[[Any], ModelSpec]
    model_types: tuple[str, ...] = ()
    # The files' tensors, by name, to the model's: for checkpoints whose tensors are named or cut otherwise
    # than the parts name and cut theirs (projections stored as one fused tensor, another prefix).  Takes and
    # returns {name: tensor}; called with the configuration before anything is checked.
    adapt_tensors: Callable[[dict, Any], dict] | None = None


ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(
    name: str,
    config_class: type[ArchitectureConfig],
    build_spec: Callable[[Any], ModelSpec],
    model_types: tuple[str, ...] = (),
    adapt_tensors: Callable[[dict, Any], dict] | None = None,
) -> Architecture:
    entry = Architecture(name, config_class, build_spec, model_types, adapt_tensors)
    ARCHITECTURES[name] = entry
    return entry


def unregister_architecture(name: str) -> None:
    ARCHITECTURES.pop(name, None)


def resolve_architecture(config_values: dict[str, Any]) -> Architecture:
    """Chooses by config.json's `architectures`, else by its `model_type`."""
    for name in config_values.get("architectures") or ():
        if name in ARCHITECTURES:
            return ARCHITECTURES[name]
    model_type = config_values.get("model_type")
    for entry in ARCHITECTURES.values():
        if model_type is not None and model_type in entry.model_types:
            return entry
    raise ConfigError(
        f"no registered architecture for architectures={config_values.get('architectures')!r}, "
        f"model_type={model_type!r} (registered: {sorted(ARCHITECTURES)})"
    )
