"""An inference engine for the Qwen2 / Qwen2.5 dense decoder on one MI355X:
from a model folder and a request's tokens to its next token."""

from . import models  # registers the architectures
from .config import CacheConfig, ConfigError, Qwen2Config, SchedulerConfig
from .cache import CacheFullError
from .engine import EngineCore, LLMEngine, ModelRunner, StepEntry
from .registry import ARCHITECTURES, register_architecture, resolve_architecture
from .sampling import GenerationConfig
from .weights import WeightsError, load_model_folder, write_model_folder

ModelConfig = Qwen2Config  # the reference's name for it (`src/llmserve/__init__.py:3`)

__version__ = "0.1.0"

__all__ = [
    "ARCHITECTURES",
    "CacheConfig",
    "CacheFullError",
    "ConfigError",
    "EngineCore",
    "GenerationConfig",
    "LLMEngine",
    "ModelRunner",
    "StepEntry",
    "WeightsError",
    "load_model_folder",
    "write_model_folder",
    "ModelConfig",
    "Qwen2Config",
    "SchedulerConfig",
    "register_architecture",
    "resolve_architecture",
]
