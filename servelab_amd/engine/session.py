"""From a model folder to a model on the device with a step function.

Reference: the first half of ``LLMEngine.__init__``
(servelab/engine/engine.py:84-111): resolve the dtype, build the model, load
the checkpoint, size and allocate the cache pool.
"""
import sys
from typing import Optional

import torch

from ..cache import CachePool
from ..parts.base import Runtime
from ..parts.model import DecoderModel, build_model_spec
from ..weights.loader import Checkpoint, load_config
from ..weights.random_init import RandomCheckpoint
from .runner import ModelRunner

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32}


FLOAT16_NOTICE = ("config.json says torch_dtype float16: this engine has bfloat16 and float32 kernels "
                  "only; the weights are converted and served in bfloat16 (8 bits of mantissa instead "
                  "of 11, a wider exponent), so logits differ from a float16 run by rounding. "
                  "Pass dtype float32 for the exact path.")


_noticed = set()


def notice_once(text: str) -> None:
    """A line on standard error, once per process."""
    if text not in _noticed:
        _noticed.add(text)
        print(f"[servelab_amd] {text}", file=sys.stderr, flush=True)


def resolve_dtype(name: str, config=None) -> torch.dtype:
    """'auto' takes config.json's torch_dtype.  There are no float16 kernels: a
    float16 checkpoint under 'auto' is served in bfloat16 and says so on
    standard error, once per process, and in the engine's ``stats()``
    (``dtype_substituted``); the reference serves it as float16
    (servelab/engine/engine.py:35-39), so logits of float16 checkpoints are
    held to no reference figure.  float16 asked for by name is refused."""
    if name in (None, "auto"):
        name = getattr(config, "dtype", "bfloat16")
        if name in ("float16", "fp16", "half"):
            notice_once(FLOAT16_NOTICE)
            name = "bfloat16"
    if name not in _DTYPES:
        raise ValueError(f"dtype must be bfloat16 or float32 (or auto), is {name!r}: "
                         "there are no kernels for other types")
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


def random_model_on_device(config, seed: int, dtype="auto", device="cuda:0", ops=None) -> DecoderModel:
    """A DecoderModel of ``config`` with seeded random weights drawn on the
    device, tensor by tensor as the parts load them; no folder is written
    (examples/run_engine.py:21-24 makes its tiny default model on the host)."""
    rt = make_runtime(resolve_dtype(dtype, config), device, ops)
    model = DecoderModel(build_model_spec(config), rt)
    model.load(RandomCheckpoint(model.spec.param_specs(), seed, rt.device, rt.act_dtype))
    return model


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
