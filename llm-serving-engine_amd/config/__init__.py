from .model import ArchitectureConfig, ConfigError, KeyReader, Qwen2Config
from .serving import CacheConfig, SchedulerConfig

__all__ = [
    "ArchitectureConfig",
    "CacheConfig",
    "ConfigError",
    "KeyReader",
    "Qwen2Config",
    "SchedulerConfig",
]
