from .model_config import ConfigError, Qwen3Config, canonical_dtype, read_config_json
from .engine_config import EngineConfig
from .registry import (Architecture, register_architecture, get_architecture,
                       architecture_of, known_architectures)

__all__ = ["ConfigError", "Qwen3Config", "canonical_dtype", "read_config_json", "EngineConfig",
           "Architecture", "register_architecture", "get_architecture", "architecture_of",
           "known_architectures"]
