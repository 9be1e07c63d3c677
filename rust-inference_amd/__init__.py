"""A small generation library for the Qwen3 dense decoder on one MI355X."""
from .api import Model, generate
from .config import Qwen3Config, load_config, register_architecture
from .errors import (CacheError, ConfigError, InferenceError, KernelError, ShapeError, UnsupportedError,
                     WeightsError)
from .sampling import SamplingParams

__all__ = ["Model", "generate", "Qwen3Config", "load_config", "register_architecture", "SamplingParams",
           "InferenceError", "ConfigError", "UnsupportedError", "WeightsError", "ShapeError", "CacheError",
           "KernelError"]
