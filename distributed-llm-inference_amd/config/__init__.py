"""Typed model configurations and the architecture registry."""

from .errors import ConfigError, MissingConfigKeyError, UnsupportedModelError
from .llama import LlamaConfig, RopeConfig
from .registry import (
    Architecture,
    load_config,
    read_config_json,
    register_architecture,
    registered_architectures,
    resolve_architecture,
    unregister_architecture,
)

__all__ = [
    "Architecture", "ConfigError", "LlamaConfig", "MissingConfigKeyError", "RopeConfig",
    "UnsupportedModelError", "load_config", "read_config_json", "register_architecture",
    "registered_architectures", "resolve_architecture", "unregister_architecture",
]
