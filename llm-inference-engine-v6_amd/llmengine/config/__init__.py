from .base import ConfigError, KeyReader, read_model_json
from .llama import LlamaConfig, RopeScaling
from .registry import (Architecture, architecture_name, known_architectures, load_config,
                       parse_config, register_architecture, resolve)

__all__ = [
    "ConfigError", "KeyReader", "read_model_json", "LlamaConfig", "RopeScaling", "Architecture",
    "architecture_name", "known_architectures", "load_config", "parse_config",
    "register_architecture", "resolve",
]
