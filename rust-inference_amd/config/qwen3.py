"""Configuration of the Qwen3 dense decoder, from its config.json keys.

Keys and defaults follow src/models/config.rs:19-56 of the reference; validation
follows :87-111.  Mixture-of-experts and quantized checkpoints are refused by name
instead of being read as a dense bfloat16 model.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar, Optional

from ..errors import ConfigError, UnsupportedError
from .base import ModelConfig, f32, whole


@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    vocab_size: int = 0
    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: Optional[int] = None          # falls back to hidden_size / heads (config.rs:75-77)
    max_position_embeddings: int = 40960    # config.rs:57-59
    rms_norm_eps: float = 1e-6              # config.rs:60-62, a 32-bit number
    rope_theta: float = 1_000_000.0         # config.rs:63-65, a 32-bit number
    tie_word_embeddings: bool = False       # config.rs:35-36: absent means untied

    ARCHITECTURE: ClassVar[str] = "Qwen3ForCausalLM"
    MODEL_TYPE: ClassVar[str] = "qwen3"
    REQUIRED: ClassVar[tuple[str, ...]] = (
        "vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
        "num_attention_heads", "num_key_value_heads",
    )

    @property
    def dim_per_head(self) -> int:
        return self.head_dim if self.head_dim else self.hidden_size // self.num_attention_heads

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        cls.require(raw)
        if int(raw.get("num_experts", 0) or 0) > 0:
            raise UnsupportedError("config.json has num_experts > 0: mixture-of-experts Qwen3 is not supported")
        if raw.get("quantization_config") is not None:
            raise UnsupportedError("config.json has a quantization_config: quantized weights are not supported")
        scaling = raw.get("rope_scaling")
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if kind not in (None, "default"):
                raise ConfigError(f"rope_scaling {scaling!r} is not supported")   # config.rs:104-109
        hd = raw.get("head_dim")
        cfg = cls(
            vocab_size=whole(raw["vocab_size"], "vocab_size", 1),
            hidden_size=whole(raw["hidden_size"], "hidden_size", 1),
            intermediate_size=whole(raw["intermediate_size"], "intermediate_size", 1),
            num_hidden_layers=whole(raw["num_hidden_layers"], "num_hidden_layers", 1),
            num_attention_heads=whole(raw["num_attention_heads"], "num_attention_heads"),
            num_key_value_heads=whole(raw["num_key_value_heads"], "num_key_value_heads"),
            head_dim=None if hd is None else whole(hd, "head_dim", 1),
            max_position_embeddings=whole(raw.get("max_position_embeddings", 40960), "max_position_embeddings", 1),
            rms_norm_eps=f32(raw.get("rms_norm_eps", 1e-6), "rms_norm_eps"),
            rope_theta=f32(raw.get("rope_theta", 1_000_000.0), "rope_theta"),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        h, hkv = self.num_attention_heads, self.num_key_value_heads
        if h == 0 or hkv == 0:
            raise ConfigError("attention heads must be non-zero")                       # config.rs:89-91
        if h % hkv != 0:
            raise ConfigError(f"{h} attention heads not divisible by {hkv} kv heads")   # config.rs:92-97
        if self.head_dim is None and self.hidden_size % h != 0:
            raise ConfigError(f"hidden_size {self.hidden_size} not divisible by {h} heads and no head_dim given")
        if self.dim_per_head % 2 != 0:
            raise ConfigError(f"head_dim {self.dim_per_head} must be even for rotary embeddings")  # config.rs:98-100
        if not self.rms_norm_eps >= 0.0:
            raise ConfigError(f"rms_norm_eps {self.rms_norm_eps} must not be negative")
        if not self.rope_theta > 0.0:
            raise ConfigError(f"rope_theta {self.rope_theta} must be positive")
