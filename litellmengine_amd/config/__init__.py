from .model_config import ConfigError, Qwen3Config, read_config_json, FULL_ATTENTION, SLIDING_ATTENTION
from .registry import (
    Architecture,
    architecture_of,
    get_architecture,
    load_config,
    register_architecture,
    registered_architectures,
)

__all__ = [
    "Architecture",
    "ConfigError",
    "Qwen3Config",
    "FULL_ATTENTION",
    "SLIDING_ATTENTION",
    "architecture_of",
    "get_architecture",
    "load_config",
    "read_config_json",
    "register_architecture",
    "registered_architectures",
]
