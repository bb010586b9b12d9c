"""Cache, scheduler and engine configuration.

Reference: servelab/config.py:75-107.  Prefix caching, eviction, offload, swap
and quantized cache formats are not part of this engine, so their fields are
gone; what remains keeps the reference's names, meanings and defaults.
"""
from dataclasses import dataclass, field
from typing import Optional

PAGE_SIZES = (16, 32, 64)


@dataclass
class CacheConfig:
    block_size: int = 16                   # tokens per page
    num_blocks: Optional[int] = None       # pages per cache group; None => from free memory
    gpu_memory_utilization: float = 0.85   # fraction of *free* device memory for the cache

    def __post_init__(self):
        if self.block_size not in PAGE_SIZES:
            raise ValueError(f"block_size must be one of {PAGE_SIZES}, is {self.block_size}")
        if self.num_blocks is not None and self.num_blocks < 1:
            raise ValueError("num_blocks must be >= 1")
        if not 0.0 < self.gpu_memory_utilization <= 1.0:
            raise ValueError("gpu_memory_utilization must be in (0, 1]")


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 64
    max_num_batched_tokens: int = 2048
    chunked_prefill: bool = True
    policy: str = "fcfs"                   # fcfs | priority | sjf-predicted (needs the engine's predictor)

    def __post_init__(self):
        if self.max_num_seqs < 1:
            raise ValueError("max_num_seqs must be >= 1")
        if self.max_num_batched_tokens < 1:
            raise ValueError("max_num_batched_tokens must be >= 1")
        if self.policy not in ("fcfs", "priority", "sjf-predicted"):
            raise ValueError(f"unknown scheduler policy: {self.policy}")


@dataclass
class EngineConfig:
    """Everything ``LLMEngine`` is built from beside the model, in one record
    (``LLMEngine.from_engine_config``; servelab/config.py:98-107)."""
    cache: CacheConfig = field(default_factory=CacheConfig)
    scheduler: SchedulerConfig = field(default_factory=SchedulerConfig)
    seed: int = 1234
    dtype: str = "auto"                    # auto (config.json's torch_dtype) | bfloat16 | float32
    device: str = "cuda:0"
    tune_products: object = False          # True, or further row counts: time the library's kernels at start-up
    capture_graphs_up_to: int = 0          # > 0: capture the decode graphs of 1..max_num_seqs requests for
                                           # contexts up to this many tokens at start-up (0: at first sight)
    run_ahead: bool = True                 # queue the next decode step before this one's tokens are read
