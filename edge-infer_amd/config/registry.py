"""One registry from an architecture's name to its configuration class and model.

The name is config.json's `architectures[0]`; `model_type` is accepted as a
second way to name the same entry (the reference's validation tool checks
`model_type == "qwen3"`, tools/validation/qwen3_reference.py:495; its runtime
takes a model-type string from the user, runtime/include/model_factory.hpp:12-37).
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Dict, Mapping, Optional


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any                       # has from_dict(), model_spec(), checkpoint_name()
    # (spec, params, dtype, device) -> model; None: engine.model.DecoderModel
    model_factory: Optional[Callable] = None
    model_types: tuple = ()


_ARCHITECTURES: Dict[str, Architecture] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_class, model_factory=None, model_types=()) -> None:
    if name in _ARCHITECTURES:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, model_factory, tuple(model_types))
    for model_type in model_types:
        _MODEL_TYPES[model_type] = name


def unregister_architecture(name: str) -> None:
    entry = _ARCHITECTURES.pop(name)
    for model_type in entry.model_types:
        _MODEL_TYPES.pop(model_type, None)


def architecture_entry(name: str) -> Optional[Architecture]:
    """The registered entry of an architecture's name, or None."""
    return _ARCHITECTURES.get(name)


def known_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(config: Mapping[str, Any]) -> Architecture:
    names = config.get("architectures") or []
    if isinstance(names, str):
        names = [names]
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
    model_type = config.get("model_type")
    if model_type in _MODEL_TYPES:
        return _ARCHITECTURES[_MODEL_TYPES[model_type]]
    raise KeyError(
        f"no registered architecture for architectures={list(names)!r}, "
        f"model_type={model_type!r}; known: {known_architectures()}")


def read_config(model_dir) -> tuple:
    """(architecture entry, typed configuration, raw dict) of a model folder."""
    path = Path(model_dir) / "config.json"
    with path.open(encoding="utf-8") as source:
        raw = json.load(source)
    if not isinstance(raw, dict):
        raise ValueError(f"{path} must hold a JSON object")
    entry = resolve_architecture(raw)
    return entry, entry.config_class.from_dict(raw), raw
