"""One registry from an architecture's name to its configuration class and its
model builder.

The reference has no registry: it checks ``model_type`` against a tuple
(servelab/config.py:50-54) and looks the q/k/v bias up by architecture
(servelab/parallel/tp_model.py:29).  Here config.json's ``architectures[0]``
(falling back to ``model_type``) selects an entry; the entry's configuration
class reads config.json and its builder turns that configuration into a
``ModelSpec`` (servelab_amd/parts/model.py) made of parts.
"""
from dataclasses import dataclass
from typing import Any, Callable, Dict


@dataclass
class Architecture:
    name: str
    config_from_hf: Callable[[Dict[str, Any], str], Any]
    build_spec: Callable[[Any], Any]


_ARCHITECTURES: Dict[str, Architecture] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_from_hf, build_spec, model_type: str = None):
    """Register (or replace) an architecture.  ``model_type`` optionally maps
    config.json's model_type to it when ``architectures`` is absent."""
    _ARCHITECTURES[name] = Architecture(name, config_from_hf, build_spec)
    if model_type:
        _MODEL_TYPES[model_type] = name


def registered_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(cfg: Dict[str, Any]) -> Architecture:
    archs = cfg.get("architectures") or []
    name = archs[0] if archs else _MODEL_TYPES.get(cfg.get("model_type", ""), None)
    if name is None or name not in _ARCHITECTURES:
        asked = archs[0] if archs else f"model_type={cfg.get('model_type')!r}"
        raise ValueError(
            f"unsupported architecture: {asked}; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]
