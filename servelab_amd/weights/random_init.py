"""Seeded random weights: a model folder from a configuration and a seed.

Reference: ``build_tiny_qwen2`` (tests/helpers_tiny_model.py:7-56) writes
config.json and seeded random tensors into a folder and
examples/run_engine.py:21-24 uses it when no model is given.  Here the set of
tensors comes from the model's own parts (so any registered architecture can be
initialised), matrices, tables and biases are N(0, std) and norm gains are
1 + N(0, norm_std); tensors are drawn in the order the model lists them from one
CPU generator, in float32, then stored in the configuration's torch_dtype.

``RandomCheckpoint`` is the same thing without the folder: it stands where a
``Checkpoint`` stands and draws each tensor on the device at the moment a part
asks for it, so a model of the 7B shape and beyond starts in seconds and no
15-150 GB file is written (the reference draws on the host and writes a folder,
which is fine for its tiny test model only).
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


class RandomCheckpoint:
    """Seeded random tensors by checkpoint name, drawn on ``device`` when asked
    for: matrices and biases N(0, std), gains 1 + N(0, norm_std).  A tensor's
    values depend on the seed and on its place in ``param_specs`` only.
    Matrices come in ``dtype``, vectors in float32 (as a loaded checkpoint's
    vectors are kept by the parts)."""

    def __init__(self, param_specs, seed: int, device, dtype: torch.dtype = torch.bfloat16,
                 std: float = 0.02, norm_std: float = 0.05):
        self.specs = dict(param_specs)
        self.seed, self.device, self.dtype = int(seed), torch.device(device), dtype
        self.std, self.norm_std = float(std), float(norm_std)
        self._index = {name: i for i, name in enumerate(self.specs)}

    def shapes(self):
        return {name: tuple(spec.shape) for name, spec in self.specs.items()}

    def __contains__(self, name: str) -> bool:
        return name in self.specs

    def get(self, name: str) -> torch.Tensor:
        spec = self.specs[name]
        gen = torch.Generator(device=self.device)
        gen.manual_seed(self.seed * 100003 + self._index[name])
        t = torch.randn(spec.shape, generator=gen, device=self.device, dtype=torch.float32)
        t = t.mul_(self.norm_std).add_(1.0) if spec.init == "gain" else t.mul_(self.std)
        return t.to(self.dtype) if len(spec.shape) > 1 else t

    def state_dict(self) -> Dict[str, torch.Tensor]:
        return {name: self.get(name) for name in self.specs}
