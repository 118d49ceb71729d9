"""Typed configurations and the architecture registry."""

from .base import ConfigError, KeyReader, ModelConfig, architecture_of, read_config_json
from .engine import (DEFAULT_BLOCK_SIZE, DEFAULT_MAX_CONCURRENT, DEFAULT_NUM_BLOCKS,
                     EngineConfig, normalize_dtype)
from .qwen2 import Qwen2Config
from .registry import (Architecture, config_from_dict, register_architecture,
                       registered_architectures, resolve_architecture, unregister_architecture)

__all__ = [
    "Architecture", "ConfigError", "DEFAULT_BLOCK_SIZE", "DEFAULT_MAX_CONCURRENT",
    "DEFAULT_NUM_BLOCKS", "EngineConfig", "KeyReader", "ModelConfig", "Qwen2Config",
    "architecture_of", "config_from_dict", "normalize_dtype", "read_config_json",
    "register_architecture", "registered_architectures", "resolve_architecture",
    "unregister_architecture",
]
