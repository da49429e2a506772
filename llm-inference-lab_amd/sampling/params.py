"""Sampling options of a request.

Field names are those of the reference's ``GenerationConfig`` (alias
``SamplingConfig``; rust/engine/src/runner/loader.rs:30-44,
rust/engine/src/types.rs:15): ``do_sample``, ``temperature``, ``top_k``,
``top_p``, ``max_new_tokens``, ``eos_token_id`` (one id or several).  The
reference runs greedy requests only and refuses the rest
(rust/engine/src/runner/model_runner.rs:615-623); here greedy and temperature
sampling run, and ``top_k`` / ``top_p`` are refused in the same way.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Optional, Sequence, Tuple, Union


@dataclasses.dataclass
class SamplingConfig:
    do_sample: Optional[bool] = None
    temperature: Optional[float] = None
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    max_new_tokens: Optional[int] = None        # the reference's default is 1 (model_runner.rs:625)
    eos_token_id: Union[None, int, Sequence[int]] = None
    seed: int = 0                               # of the request's random stream

    def validate(self) -> None:
        if self.top_k is not None or self.top_p is not None:
            raise ValueError("only greedy and temperature sampling are supported "
                             "(top_k and top_p must be unset)")
        if self.temperature is not None and not self.temperature >= 0.0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if self.max_new_tokens is not None and self.max_new_tokens < 0:
            raise ValueError(f"max_new_tokens must be >= 0, got {self.max_new_tokens}")

    @property
    def effective_temperature(self) -> float:
        """0 means greedy: no sampling asked for, or a temperature of 0."""
        if self.do_sample is False:
            return 0.0
        if self.temperature is None:
            return 1.0 if self.do_sample else 0.0
        return float(self.temperature)

    @property
    def new_tokens(self) -> int:
        return 1 if self.max_new_tokens is None else int(self.max_new_tokens)

    def eos_ids(self, model_default: Sequence[int] = ()) -> Tuple[int, ...]:
        """The request's own ids if it names any, else the model's."""
        if self.eos_token_id is None:
            return tuple(model_default)
        if isinstance(self.eos_token_id, int):
            return (self.eos_token_id,)
        return tuple(int(e) for e in self.eos_token_id)


def _check_generation_field(path: str, key: str, value):
    """One field of ``generation_config.json``, type-checked; the error names the key."""
    from ..config.errors import ConfigError

    def bad(expected):
        return ConfigError(f"{path}: '{key}' must be {expected}, got {value!r}")
    if value is None:
        return None
    if key == "do_sample":
        if not isinstance(value, bool):
            raise bad("true or false")
        return value
    if key in ("temperature", "top_p"):
        if isinstance(value, bool) or not isinstance(value, (int, float)) or not value >= 0:
            raise bad("a number >= 0")
        return float(value)
    if key in ("top_k", "max_new_tokens"):
        if isinstance(value, bool) or not isinstance(value, int) or value < 0:
            raise bad("an integer >= 0")
        return value
    if key == "eos_token_id":
        ids = value if isinstance(value, list) else [value]
        if not all(isinstance(i, int) and not isinstance(i, bool) and i >= 0 for i in ids):
            raise bad("a token id or a list of token ids")
        return value if isinstance(value, int) else [int(i) for i in ids]
    return value


def read_generation_config(model_dir: str) -> Optional[SamplingConfig]:
    """The optional ``generation_config.json`` of a model folder, or None if there is
    none (rust/engine/src/runner/loader.rs:199-205).  The reference's fields are read
    (loader.rs:30-44), every other key of the file is ignored."""
    path = os.path.join(model_dir, "generation_config.json")
    if not os.path.isfile(path):
        return None
    from ..config.errors import ConfigError
    with open(path, "r", encoding="utf-8") as f:
        try:
            raw = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: a JSON object is expected")
    known = ("do_sample", "temperature", "top_k", "top_p", "max_new_tokens", "eos_token_id")
    return SamplingConfig(**{k: _check_generation_field(path, k, raw[k]) for k in known if k in raw})
