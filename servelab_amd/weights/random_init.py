"""Seeded random weights: a model folder from a configuration and a seed.

Reference: ``build_tiny_qwen2`` (tests/helpers_tiny_model.py:7-56) writes
config.json and seeded random tensors into a folder and
examples/run_engine.py:21-24 uses it when no model is given.  Here the set of
tensors comes from the model's own parts (so any registered architecture can be
initialised), matrices, tables and biases are N(0, std) and norm gains are
1 + N(0, norm_std); tensors are drawn in the order the model lists them from one
CPU generator, in float32, then stored in the configuration's torch_dtype.
"""
import json
import os
from typing import Dict

import torch

from .safetensors_io import write_safetensors

_STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def random_tensors(param_specs, seed: int, std: float = 0.02,
                   norm_std: float = 0.05) -> Dict[str, torch.Tensor]:
    """{checkpoint name: float32 tensor} for ``param_specs`` ({name: ParamSpec})."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    out = {}
    for name, spec in param_specs.items():
        noise = torch.randn(spec.shape, generator=gen, dtype=torch.float32)
        out[name] = 1.0 + noise * norm_std if spec.init == "gain" else noise * std
    return out


def write_random_model(config, folder: str, seed: int = 0, std: float = 0.02,
                       norm_std: float = 0.05) -> str:
    """Write ``folder``/config.json and model.safetensors; returns the folder."""
    from ..parts.model import build_model_spec
    spec = build_model_spec(config)
    tensors = random_tensors(spec.param_specs(), seed, std, norm_std)
    store = _STORE.get(getattr(config, "dtype", "float32"), torch.float32)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_hf(), f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: t.to(store) for n, t in tensors.items()},
                      metadata={"format": "pt", "seed": seed})
    return folder
