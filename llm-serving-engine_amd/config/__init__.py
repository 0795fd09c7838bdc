from .model import ArchitectureConfig, ConfigError, KeyReader, Qwen2Config
from .dafutar import DafutarConfig
from .katenex import KatenexConfig
from .sozavik import SozavikConfig
from .vagozen import VagozenConfig
from .serving import CacheConfig, SchedulerConfig

__all__ = [
    "ArchitectureConfig",
    "CacheConfig",
    "ConfigError",
    "DafutarConfig",
    "KatenexConfig",
    "KeyReader",
    "Qwen2Config",
    "SchedulerConfig",
    "SozavikConfig",
    "VagozenConfig",
]
