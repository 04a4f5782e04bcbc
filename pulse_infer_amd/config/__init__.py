from .base import ConfigError, JsonReader, ModelConfig
from .registry import (ArchitectureEntry, config_from_dict, load_config, lookup_architecture,
                       register_architecture, registered_architectures, unregister_architecture)
from .qwen3 import Qwen3Config

register_architecture(Qwen3Config.architecture, Qwen3Config, replace=True)

__all__ = [
    "ConfigError", "JsonReader", "ModelConfig", "ArchitectureEntry", "config_from_dict", "load_config",
    "lookup_architecture", "register_architecture", "registered_architectures",
    "unregister_architecture", "Qwen3Config",
]
