"""Typed configuration of the Qwen2 dense decoder, read from ``config.json``.

Keys and their meaning follow the reference's ``Qwen2Config``
(rust/engine/src/runner/model/qwen2/engine.rs:197-216) and its load-time
validation (engine.rs:260-288).  The reference fixes ``head_dim`` at 64 and
rejects sliding windows; here ``head_dim``, ``sliding_window`` and
``max_window_layers`` are read as well, with the defaults the checkpoint format
gives them.
"""
from __future__ import annotations

import dataclasses
import json
import math
import os
from typing import Any, Dict, List, Optional, Tuple

from .errors import ConfigError


def _require(raw: Dict[str, Any], key: str, kind, where: str):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return _typed(raw[key], key, kind, where)


def _typed(value, key: str, kind, where: str):
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"{where}: key '{key}' must be an integer, got {value!r}")
        return value
    if kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{where}: key '{key}' must be a number, got {value!r}")
        return float(value)
    if kind is bool:
        if not isinstance(value, bool):
            raise ConfigError(f"{where}: key '{key}' must be true or false, got {value!r}")
        return value
    if kind is str:
        if not isinstance(value, str):
            raise ConfigError(f"{where}: key '{key}' must be a string, got {value!r}")
        return value
    raise AssertionError(kind)


@dataclasses.dataclass(frozen=True)
class Qwen2Config:
    """Every size and constant of a Qwen2 decoder; nothing here has a default
    that stands for a model size."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: int = 0
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Qwen2ForCausalLM"
    model_type: str = "qwen2"

    ARCHITECTURE = "Qwen2ForCausalLM"
    MODEL_TYPE = "qwen2"

    # ------------------------------------------------------------------ read
    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "Qwen2Config":
        model_type = _typed(raw.get("model_type", "qwen2"), "model_type", str, where)
        if model_type != "qwen2":
            raise ConfigError(f"{where}: model_type must be 'qwen2', got '{model_type}'")
        archs = raw.get("architectures") or [cls.ARCHITECTURE]
        hidden = _require(raw, "hidden_size", int, where)
        heads = _require(raw, "num_attention_heads", int, where)
        kv_heads = raw.get("num_key_value_heads")
        kv_heads = heads if kv_heads is None else _typed(kv_heads, "num_key_value_heads", int, where)
        head_dim = raw.get("head_dim")
        if head_dim is None:
            if heads <= 0 or hidden % heads != 0:
                raise ConfigError(
                    f"{where}: hidden_size {hidden} is not a multiple of num_attention_heads "
                    f"{heads} and no 'head_dim' is given")
            head_dim = hidden // heads
        else:
            head_dim = _typed(head_dim, "head_dim", int, where)
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError(f"{where}: 'rope_scaling' is not supported (must be null)")
        use_window = _typed(raw.get("use_sliding_window", False), "use_sliding_window", bool, where)
        window = raw.get("sliding_window")
        if window is not None:
            window = _typed(window, "sliding_window", int, where)
        layers = _require(raw, "num_hidden_layers", int, where)
        max_window_layers = raw.get("max_window_layers")
        max_window_layers = layers if max_window_layers is None else _typed(
            max_window_layers, "max_window_layers", int, where)
        eos = raw.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, list):
            eos_ids = tuple(_typed(e, "eos_token_id", int, where) for e in eos)
        else:
            eos_ids = (_typed(eos, "eos_token_id", int, where),)
        cfg = cls(
            vocab_size=_require(raw, "vocab_size", int, where),
            hidden_size=hidden,
            intermediate_size=_require(raw, "intermediate_size", int, where),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=_require(raw, "rms_norm_eps", float, where),
            rope_theta=_typed(raw.get("rope_theta", 10000.0), "rope_theta", float, where),
            max_position_embeddings=_require(raw, "max_position_embeddings", int, where),
            tie_word_embeddings=_typed(raw.get("tie_word_embeddings", False),
                                       "tie_word_embeddings", bool, where),
            hidden_act=_typed(raw.get("hidden_act", "silu"), "hidden_act", str, where),
            use_sliding_window=use_window,
            sliding_window=window,
            max_window_layers=max_window_layers,
            eos_token_ids=eos_ids,
            architecture=str(archs[0]),
            model_type=model_type,
        )
        cfg.validate(where)
        return cfg

    @classmethod
    def from_dir(cls, model_dir: str) -> "Qwen2Config":
        path = os.path.join(model_dir, "config.json")
        with open(path, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f), where=path)

    # -------------------------------------------------------------- validate
    def validate(self, where: str = "config") -> None:
        def positive(name):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{where}: '{name}' must be positive, got {getattr(self, name)}")
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim",
                     "max_position_embeddings"):
            positive(name)
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"{where}: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"{where}: head_dim {self.head_dim} must be even for rotary pairs")
        if not (math.isfinite(self.rms_norm_eps) and self.rms_norm_eps > 0):
            raise ConfigError(f"{where}: rms_norm_eps must be finite and > 0, got {self.rms_norm_eps}")
        if not (math.isfinite(self.rope_theta) and self.rope_theta > 0):
            raise ConfigError(f"{where}: rope_theta must be finite and > 0, got {self.rope_theta}")
        if self.hidden_act != "silu":
            raise ConfigError(f"{where}: hidden_act must be 'silu', got '{self.hidden_act}'")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window <= 0:
                raise ConfigError(
                    f"{where}: use_sliding_window is true but 'sliding_window' is "
                    f"{self.sliding_window!r}")
            if self.max_window_layers < 0:
                raise ConfigError(f"{where}: max_window_layers must be >= 0")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab_size:
                raise ConfigError(f"{where}: eos_token_id {e} is outside the vocabulary")

    # ----------------------------------------------------------------- derive
    def layer_window(self, layer: int) -> Optional[int]:
        """Window of a layer in tokens (the query's own position counts), or
        ``None`` for full causal attention: layers with index >=
        ``max_window_layers`` are windowed when ``use_sliding_window`` is set."""
        if self.use_sliding_window and self.sliding_window is not None \
                and layer >= self.max_window_layers:
            return int(self.sliding_window)
        return None

    def to_dict(self) -> Dict[str, Any]:
        """The ``config.json`` form of this configuration."""
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
            "rope_scaling": None,
        }
        if len(self.eos_token_ids) == 1:
            out["eos_token_id"] = self.eos_token_ids[0]
        elif self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    def parameter_count(self) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        q = self.num_attention_heads * self.head_dim
        kv = self.num_key_value_heads * self.head_dim
        per_layer = q * h + q + 2 * (kv * h + kv) + h * q + 3 * h * i + 2 * h
        head = 0 if self.tie_word_embeddings else v * h
        return v * h + self.num_hidden_layers * per_layer + h + head
