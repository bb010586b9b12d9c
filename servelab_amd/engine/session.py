"""From a model folder to a model on the device with a step function.

Reference: the first half of ``LLMEngine.__init__``
(servelab/engine/engine.py:84-111): resolve the dtype, build the model, load
the checkpoint, size and allocate the cache pool.
"""
from typing import Optional

import torch

from ..cache import CachePool
from ..parts.base import Runtime
from ..parts.model import DecoderModel, build_model_spec
from ..weights.loader import Checkpoint, load_config
from .runner import ModelRunner

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32}


def resolve_dtype(name: str, config=None) -> torch.dtype:
    """'auto' takes config.json's torch_dtype; float16 checkpoints are served
    in bfloat16 (weights are kept in bfloat16)."""
    if name in (None, "auto"):
        name = getattr(config, "dtype", "bfloat16")
        if name == "float16":
            name = "bfloat16"
    if name not in _DTYPES:
        raise ValueError(f"dtype must be bfloat16 or float32, is {name!r}")
    return _DTYPES[name]


def make_runtime(dtype: torch.dtype, device="cuda:0", ops=None) -> Runtime:
    if ops is None:
        from ..kernels import HipOps
        ops = HipOps(dtype, device)
    return Runtime(ops, device, dtype)


def load_model_on_device(folder: str, dtype="auto", device="cuda:0", ops=None, config=None):
    """(configuration, DecoderModel) with the folder's weights on the device."""
    config = config or load_config(folder)
    rt = make_runtime(resolve_dtype(dtype, config), device, ops)
    model = DecoderModel(build_model_spec(config), rt)
    model.load(Checkpoint(folder))
    return config, model


def default_num_pages(model: DecoderModel, page_size: int, utilization: float) -> int:
    """free bytes * utilization / bytes per page index over all paged streams,
    at least 16 (servelab/engine/engine.py:273-288)."""
    itemsize = torch.empty((), dtype=model.rt.act_dtype).element_size()
    per_page = CachePool.bytes_per_page(model.spec.stream_specs(), page_size, itemsize)
    if model.rt.device.type != "cuda" or per_page == 0:
        return 4096
    free, _ = torch.cuda.mem_get_info(model.rt.device)
    return max(16, int(free * utilization / per_page))


def make_runner(model: DecoderModel, num_pages: Optional[int], page_size: int = 16,
                max_num_seqs: int = 64, utilization: float = 0.85) -> ModelRunner:
    if not num_pages:
        num_pages = default_num_pages(model, page_size, utilization)
    return ModelRunner(model, num_pages, page_size, max_num_seqs)
