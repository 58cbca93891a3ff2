from .model import ArchitectureConfig, ConfigError, KeyReader, Qwen2Config
from .dafutar import DafutarConfig
from .serving import CacheConfig, SchedulerConfig

__all__ = [
    "ArchitectureConfig",
    "CacheConfig",
    "ConfigError",
    "DafutarConfig",
    "KeyReader",
    "Qwen2Config",
    "SchedulerConfig",
]
