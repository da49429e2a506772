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
    # (config, expected tensor specs, seed, dtype) -> (name, tensor) pairs: the architecture's
    # own way of drawing random weights; None: every tensor as its TensorSpec.init says
    random_init: Callable[..., Any] = None
    # what the command line needs beside the model: "{prompt}" in ``chat_template`` is
    # replaced by the user's text before it is tokenised (None: the text as it is)
    chat_template: str = None


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class, build_spec, random_init=None,
                          replace: bool = False, chat_template: str = None) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec, random_init, chat_template)


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
    """The entry that ``architectures[0]`` names.  A configuration without that key (one
    written by hand for the random-weights mode) is matched by its ``model_type`` against
    the ``MODEL_TYPE`` of the registered configuration classes."""
    archs = raw.get("architectures")
    if archs is None and isinstance(raw.get("model_type"), str):
        hits = [a for a in _ARCHITECTURES.values()
                if getattr(a.config_class, "MODEL_TYPE", None) == raw["model_type"]]
        if len(hits) == 1:
            return hits[0]
        raise ConfigError(f"{where}: no key 'architectures', and model_type '{raw['model_type']}' names "
                          f"{len(hits)} of the registered architectures "
                          f"({', '.join(registered_architectures())})")
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
