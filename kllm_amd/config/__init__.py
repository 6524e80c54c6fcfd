from .base import ConfigError, ModelConfig, read_config_json
from .llama import LlamaConfig
from .registry import (Architecture, register_architecture, unregister_architecture,
                       registered_architectures, resolve_architecture, config_from_dict,
                       load_config)

__all__ = [
    "ConfigError", "ModelConfig", "read_config_json", "LlamaConfig", "Architecture",
    "register_architecture", "unregister_architecture", "registered_architectures",
    "resolve_architecture", "config_from_dict", "load_config",
]
