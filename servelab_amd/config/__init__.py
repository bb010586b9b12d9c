from .model import ConfigError, Qwen2Config, read_key
from .engine import CacheConfig, SchedulerConfig, EngineConfig, PAGE_SIZES
from .registry import (Architecture, register_architecture, registered_architectures,
                       resolve_architecture)

# reference name for the model configuration (servelab/config.py:10)
ModelConfig = Qwen2Config
