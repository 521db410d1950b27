from .base import ConfigError, ModelConfig, read_config_json
from .gpt2 import GPT2Config
from .registry import (
    Architecture,
    architecture_name,
    config_from_dict,
    get_architecture,
    load_config,
    register_architecture,
    registered_architectures,
)

__all__ = [
    "Architecture",
    "ConfigError",
    "GPT2Config",
    "ModelConfig",
    "architecture_name",
    "config_from_dict",
    "get_architecture",
    "load_config",
    "read_config_json",
    "register_architecture",
    "registered_architectures",
]
