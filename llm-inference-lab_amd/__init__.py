"""A small, whole inference engine for one AMD MI355X (gfx950)."""
from . import architectures  # noqa: F401
from .config import (ConfigError, WeightError, UnsupportedSizeError, Qwen2Config, ModelSpec,
                     PartSpec, BlockSpec, ScheduleEntry, register_architecture,
                     registered_architectures, read_config)
from .parts import register_part
from .engine import Engine, StepEntry, write_random_model

__all__ = [
    "ConfigError", "WeightError", "UnsupportedSizeError", "Qwen2Config", "ModelSpec", "PartSpec",
    "BlockSpec", "ScheduleEntry", "register_architecture", "registered_architectures",
    "read_config", "register_part", "Engine", "StepEntry", "write_random_model",
]
