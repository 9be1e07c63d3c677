from . import attention, block, feed_forward, norm, position, qwen3  # noqa: F401  (registers the parts)
from .base import Embedding, FeedForward, Head, Mixer, Norm, Part, PositionEncoding
from .block import PreNormBlock, ResidualStream
from .context import StepContext
from .model import DecoderModel, expected_tensors, load_model, load_model_plain, random_model
from .registry import build_part, part_class, register_part, registered
from .runtime import Runtime
from .spec import LayerSpec, ModelSpec, PartSpec, Run

__all__ = ["Embedding", "Head", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding", "PreNormBlock", "ResidualStream",
           "StepContext", "DecoderModel", "expected_tensors", "load_model", "load_model_plain", "random_model", "build_part",
           "part_class", "register_part", "registered", "Runtime", "LayerSpec", "ModelSpec", "PartSpec", "Run"]
