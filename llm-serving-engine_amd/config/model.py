"""Typed model configurations read from an architecture's own config.json keys.

The reference reads a flat dict into one frozen dataclass with defaults for
every size (`src/llmserve/config.py:10-62`).  Here sizes have no defaults: a key
that config.json must give and does not is an error that names the key.
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass, fields
from pathlib import Path
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A config.json that the architecture cannot be built from."""


_MISSING = object()


class KeyReader:
    """Reads typed values out of a config dict and remembers which keys were used."""

    def __init__(self, values: dict[str, Any], where: str) -> None:
        self.values = dict(values)
        self.where = where
        self.used: set[str] = set()

    def _get(self, names: tuple[str, ...], default: Any) -> Any:
        for name in names:
            if name in self.values and self.values[name] is not None:
                self.used.add(name)
                return self.values[name]
        if default is _MISSING:
            raise ConfigError(f"{self.where}: required key {names[0]!r} is missing")
        return default

    def integer(self, *names: str, default: Any = _MISSING, minimum: int = 1) -> int:
        value = self._get(names, default)
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"{self.where}: {names[0]!r} must be an integer, got {value!r}")
        if value < minimum:
            raise ConfigError(f"{self.where}: {names[0]!r} must be >= {minimum}, got {value}")
        return value

    def number(self, *names: str, default: Any = _MISSING) -> float:
        value = self._get(names, default)
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{self.where}: {names[0]!r} must be a number, got {value!r}")
        return float(value)

    def boolean(self, *names: str, default: Any = _MISSING) -> bool:
        value = self._get(names, default)
        if not isinstance(value, bool):
            raise ConfigError(f"{self.where}: {names[0]!r} must be true or false, got {value!r}")
        return value

    def choice(self, *names: str, choices: tuple[str, ...], default: Any = _MISSING) -> str:
        value = self._get(names, default)
        if value not in choices:
            raise ConfigError(f"{self.where}: {names[0]!r} must be one of {choices}, got {value!r}")
        return value

    def optional(self, name: str) -> Any:
        value = self.values.get(name)
        if value is not None:
            self.used.add(name)
        return value


@dataclass(frozen=True)
class ArchitectureConfig:
    """Base of every architecture's typed configuration."""

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "ArchitectureConfig":
        raise NotImplementedError

    @classmethod
    def from_json_file(cls, path: str | Path) -> "ArchitectureConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    @classmethod
    def from_yaml(cls, path: str | Path) -> "ArchitectureConfig":
        import yaml

        with Path(path).open() as handle:
            return cls.from_dict(yaml.safe_load(handle))

    def to_dict(self) -> dict[str, Any]:
        return asdict(self)

    def to_config_json(self) -> dict[str, Any]:
        """The dict that `from_dict` reads back to an equal configuration."""
        raise NotImplementedError


@dataclass(frozen=True)
class Qwen2Config(ArchitectureConfig):
    """Qwen2 / Qwen2.5 dense decoder.

    Field names follow the reference's `ModelConfig` (`config.py:10-22`); the
    config.json keys `num_hidden_layers` and `max_seq_len` are accepted as the
    reference accepts them (`config.py:46-54`).  Additions: an explicit
    `head_dim` (the reference derives `hidden_size // num_attention_heads`,
    `config.py:30-32`, which stays the default), the sliding-window keys of
    Qwen2's config.json (the reference drops them silently), and
    `rope_pairing`.  `attention_bias` and `tie_word_embeddings` default to True
    when absent, as in the reference (`config.py:21-22`), and the rotation is the
    reference's unless the folder comes from transformers (see `rope_pairing`).
    """

    architecture: ClassVar[str] = "Qwen2ForCausalLM"
    model_type: ClassVar[str] = "qwen2"

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    attention_bias: bool = True
    tie_word_embeddings: bool = True
    # "adjacent": pairs (2j, 2j+1), the rotation the reference applies
    # (`model.py:39-42`), and so the default.  "half": pairs (j, j + D/2), the
    # layout of published Qwen2 checkpoints; `from_dict` chooses it for a
    # config.json that transformers wrote (it carries `transformers_version`)
    # unless `rope_pairing` says otherwise.  The two agree after permuting each
    # head's q/k rows.
    rope_pairing: str = "adjacent"
    # Layers with index >= max_window_layers see only the last `sliding_window`
    # keys when use_sliding_window is set; the others see all of them.
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int | None = None

    def __post_init__(self) -> None:
        # `config.py:24-28`
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError("num_attention_heads must be divisible by num_key_value_heads")
        if self.head_dim % 2:
            raise ConfigError("head_dim must be even for rotary position encoding")
        if self.rope_pairing not in ("half", "adjacent"):
            raise ConfigError("rope_pairing must be 'half' or 'adjacent'")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window < 1:
                raise ConfigError("use_sliding_window needs a positive sliding_window")
            if self.max_window_layers is None:
                raise ConfigError("use_sliding_window needs max_window_layers")

    def layer_window(self, index: int) -> int | None:
        if self.use_sliding_window and index >= self.max_window_layers:
            return self.sliding_window
        return None

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "Qwen2Config":
        reader = KeyReader(values, "Qwen2 config")
        model_type = reader.optional("model_type")
        if model_type is not None and model_type != cls.model_type:
            # `checkpoint.py:35-36`
            raise ConfigError(f"Qwen2 config: model_type is {model_type!r}, not 'qwen2'")
        hidden = reader.integer("hidden_size")
        heads = reader.integer("num_attention_heads")
        if "head_dim" not in values and hidden % heads:
            raise ConfigError("hidden_size must be divisible by num_attention_heads")
        scaling = reader.optional("rope_scaling")
        if scaling:
            raise ConfigError(f"Qwen2 config: rope_scaling {scaling!r} is not supported")
        activation = reader.optional("hidden_act")
        if activation not in (None, "silu"):
            raise ConfigError(f"Qwen2 config: hidden_act {activation!r} is not supported")
        use_window = reader.boolean("use_sliding_window", default=False)
        layers = reader.integer("num_hidden_layers", "num_layers")
        return cls(
            vocab_size=reader.integer("vocab_size"),
            hidden_size=hidden,
            intermediate_size=reader.integer("intermediate_size"),
            num_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=reader.integer("num_key_value_heads"),
            head_dim=reader.integer("head_dim", default=hidden // heads),
            max_position_embeddings=reader.integer("max_position_embeddings", "max_seq_len"),
            rope_theta=reader.number("rope_theta"),
            rms_norm_eps=reader.number("rms_norm_eps"),
            attention_bias=reader.boolean("attention_bias", default=True),
            tie_word_embeddings=reader.boolean("tie_word_embeddings", default=True),
            rope_pairing=reader.choice(
                "rope_pairing",
                choices=("half", "adjacent"),
                default="half" if "transformers_version" in values else "adjacent",
            ),
            use_sliding_window=use_window,
            sliding_window=reader.integer("sliding_window") if use_window else None,
            max_window_layers=reader.integer("max_window_layers", minimum=0) if use_window else None,
        )

    def to_config_json(self) -> dict[str, Any]:
        values = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "hidden_act": "silu",
            "torch_dtype": "bfloat16",
        }
        for item in fields(self):
            key = "num_hidden_layers" if item.name == "num_layers" else item.name
            if getattr(self, item.name) is not None:  # an option that is off has no key (readers that check keys strictly refuse null)
                values[key] = getattr(self, item.name)
        return values
