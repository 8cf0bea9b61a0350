from .model_config import ArchConfig, ConfigError, LlamaConfig, RopeScaling, read_config_json
from .registry import (Architecture, get_architecture, load_model_config, register_architecture,
                       registered_architectures, resolve_architecture, unregister_architecture)

__all__ = ["ArchConfig", "ConfigError", "LlamaConfig", "RopeScaling", "read_config_json", "Architecture",
           "get_architecture", "load_model_config", "register_architecture", "registered_architectures",
           "resolve_architecture", "unregister_architecture"]
