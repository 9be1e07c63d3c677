from .base import ModelConfig, read_config_json
from .qwen3 import Qwen3Config
from .registry import (Architecture, config_from_dict, known_architectures, load_config,
                       register_architecture, resolve_architecture)

__all__ = ["ModelConfig", "Qwen3Config", "Architecture", "read_config_json", "config_from_dict",
           "known_architectures", "load_config", "register_architecture", "resolve_architecture"]
