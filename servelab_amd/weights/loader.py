"""Model folder -> (configuration, tensors by checkpoint name).

Reference contract: ``load_model(path) -> (ModelConfig, state_dict)``
(servelab/engine/engine.py:87, examples/run_engine.py:39-40); the body is not
in the reference's tree.  Names are the checkpoint's own; a tensor keeps
bfloat16 (float16 becomes bfloat16), 32-bit floats stay 32-bit, integer tables
become int32.
"""
import json
import os
from typing import Any, Dict, List, Tuple

import torch

from ..config import resolve_architecture
from .safetensors_io import SafetensorsFile


class WeightError(RuntimeError):
    """The checkpoint does not hold the tensors the model needs."""


def keep_dtype(t: torch.Tensor) -> torch.Tensor:
    """The dtype a loaded tensor is kept in."""
    if t.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return t
    if t.dtype == torch.float16:
        return t.to(torch.bfloat16)
    if t.dtype == torch.float64:
        return t.to(torch.float32)
    if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8, torch.bool):
        return t.to(torch.int32)
    raise WeightError(f"dtype {t.dtype} cannot be kept")


class Checkpoint:
    """All tensors of a model folder, by name, over one or several files."""

    def __init__(self, folder: str):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        self._where: Dict[str, SafetensorsFile] = {}
        if os.path.exists(index):
            with open(index, encoding="utf-8") as f:
                weight_map = json.load(f)["weight_map"]
            files: Dict[str, SafetensorsFile] = {}
            for name, fname in weight_map.items():
                if fname not in files:
                    files[fname] = SafetensorsFile(os.path.join(folder, fname))
                if name not in files[fname].entries:
                    raise WeightError(f"{index}: '{name}' is not in {fname}")
                self._where[name] = files[fname]
        elif os.path.exists(single):
            f = SafetensorsFile(single)
            for name in f.names():
                self._where[name] = f
        else:
            raise WeightError(
                f"{folder}: neither model.safetensors nor model.safetensors.index.json")

    def shapes(self) -> Dict[str, Tuple[int, ...]]:
        return {n: f.shape(n) for n, f in self._where.items()}

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def get(self, name: str) -> torch.Tensor:
        """The tensor in the dtype it is kept in (a view or a converted copy)."""
        return keep_dtype(self._where[name].tensor(name))

    def state_dict(self) -> Dict[str, torch.Tensor]:
        return {n: self.get(n) for n in self._where}


def ignorable(name: str) -> bool:
    """Names a checkpoint may carry that no part owns: rotary tables
    (servelab/parallel/tp_model.py:104, servelab/parallel/layers.py:247)."""
    return name.endswith("rotary_emb.inv_freq")


def check_tensors(expected: Dict[str, Tuple[int, ...]],
                  found: Dict[str, Tuple[int, ...]],
                  optional: List[str] = ()) -> None:
    """One error that lists every missing tensor, every unexpected tensor and
    every wrong shape.  ``optional`` names may be present without being used
    (a stray lm_head.weight beside tied embeddings,
    servelab/parallel/tp_model.py:112-113).

    Decision: an unexpected tensor is fatal, like a missing one.  The reference
    prints the names it did not use and goes on (servelab/engine/engine.py:88-90);
    here a tensor that no part owns means the folder holds another model than
    config.json describes (further layers, an adapter, a bias the configuration
    switched off), and serving it would give logits nobody asked for.  The only
    names let through are those of ``ignorable`` and ``optional``."""
    missing = sorted(n for n in expected if n not in found)
    unexpected = sorted(n for n in found
                        if n not in expected and n not in optional and not ignorable(n))
    wrong = sorted((n, tuple(expected[n]), tuple(found[n])) for n in expected
                   if n in found and tuple(found[n]) != tuple(expected[n]))
    if not (missing or unexpected or wrong):
        return
    lines = ["checkpoint does not match the model:"]
    if missing:
        lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shape ({len(wrong)}): " + ", ".join(
            f"{n} expected {list(e)} found {list(f)}" for n, e, f in wrong))
    raise WeightError("\n".join(lines))


def read_config(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.exists(path):
        raise WeightError(f"{folder}: no config.json")
    with open(path, encoding="utf-8") as f:
        return json.load(f)


def load_config(folder: str):
    """The typed configuration of a model folder, through the registry."""
    raw = read_config(folder)
    arch = resolve_architecture(raw)
    return arch.config_from_hf(raw, folder)


def load_model(folder: str):
    """(configuration, {checkpoint name: tensor}) — the reference's entry
    (servelab/engine/engine.py:87)."""
    config = load_config(folder)
    return config, Checkpoint(folder).state_dict()
