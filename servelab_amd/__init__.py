"""servelab_amd: a one-GPU MI355X inference engine for the Qwen2 dense decoder.

From a model folder (config.json + safetensors, or seeded random weights) to
generated tokens: typed configuration and an architecture registry, a weight
loader keyed by checkpoint names, models assembled from parts, a paged cache
manager, one step function over packed batches, a continuous-batching
scheduler, sampling, and hand-written HIP kernels for gfx950.
"""
from . import models as _models  # registers the architectures  # noqa: F401
from .config import (CacheConfig, ConfigError, EngineConfig, ModelConfig, Qwen2Config,
                     SchedulerConfig, register_architecture)
from .weights import WeightError, load_config, load_model, write_random_model
from .engine import LLMEngine, RequestOutput, SamplingParams

__all__ = ["CacheConfig", "ConfigError", "EngineConfig", "ModelConfig", "Qwen2Config",
           "SchedulerConfig", "register_architecture", "WeightError", "load_config",
           "load_model", "write_random_model", "LLMEngine", "RequestOutput", "SamplingParams"]
