from .engine_config import EngineConfig
from .model_config import (
    ConfigError,
    normalise_dtype_name,
    read_architecture,
    read_config_json,
)
from .qwen3 import Qwen3Config
from .registry import (
    ArchitectureEntry,
    config_from_dict,
    register_architecture,
    resolve_architecture,
    supported_architectures,
    unregister_architecture,
)

__all__ = [
    "ArchitectureEntry",
    "ConfigError",
    "EngineConfig",
    "Qwen3Config",
    "config_from_dict",
    "normalise_dtype_name",
    "read_architecture",
    "read_config_json",
    "register_architecture",
    "resolve_architecture",
    "supported_architectures",
    "unregister_architecture",
]
