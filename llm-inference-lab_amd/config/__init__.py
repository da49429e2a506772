from .errors import ConfigError, WeightError, UnsupportedSizeError
from .spec import PartSpec, BlockSpec, ScheduleEntry, ModelSpec
from .registry import (register_architecture, unregister_architecture, get_architecture,
                       registered_architectures, architecture_of, read_config, Architecture)
from .qwen2 import Qwen2Config

__all__ = [
    "ConfigError", "WeightError", "UnsupportedSizeError", "PartSpec", "BlockSpec",
    "ScheduleEntry", "ModelSpec", "register_architecture", "unregister_architecture",
    "get_architecture", "registered_architectures", "architecture_of", "read_config",
    "Architecture", "Qwen2Config",
]
