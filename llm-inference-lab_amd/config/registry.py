"""One registry from an architecture's name to its configuration class and
its builder.

``architectures[0]`` of ``config.json`` selects the entry.  The reference has
no such table (its model type is a compile-time generic,
rust/engine/src/runner/model_runner.rs:140-149, and only ``model_type ==
"qwen2"`` is checked, rust/engine/src/runner/model/qwen2/engine.rs:260).
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Callable, Dict

from .errors import ConfigError
from .spec import ModelSpec


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any                         # has from_dict(raw, where) and to_dict()
    build_spec: Callable[[Any], ModelSpec]    # typed config -> ModelSpec
    random_init: Callable[..., Dict[str, Any]] = None   # (config, seed, dtype) -> tensors


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class, build_spec, random_init=None,
                          replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec, random_init)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"unknown architecture '{name}'; registered: {', '.join(registered_architectures())}"
        ) from None


def architecture_of(raw: Dict[str, Any], where: str = "config.json") -> Architecture:
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, list) or not isinstance(archs[0], str):
        raise ConfigError(f"{where}: key 'architectures' must be a non-empty list of names")
    return get_architecture(archs[0])


def read_config(model_dir: str):
    """Read ``config.json`` of a model folder; returns (architecture, typed config)."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file")
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    arch = architecture_of(raw, path)
    return arch, arch.config_class.from_dict(raw, where=path)
