"""Qwen3 dense as a list of parts (the reference: src/models/qwen3.rs).

Every layer: RMSNorm, grouped-query attention with per-head q/k RMSNorm and
rotate-half rotary encoding over all keys, RMSNorm, SwiGLU feed-forward, pre-norm
arrangement; tensor names as in the checkpoint (src/models/qwen3.rs:62-67, :106-108,
:157, :170-172, :184-186).
"""
from __future__ import annotations

from ..config import Qwen3Config, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, Run


def qwen3_spec(cfg: Qwen3Config) -> ModelSpec:
    d, dh, eps = cfg.hidden_size, cfg.dim_per_head, cfg.rms_norm_eps
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(
            mixer_norm=PartSpec("rmsnorm", {"dim": d, "eps": eps, "name": p + "input_layernorm.weight"}),
            mixer=PartSpec("attention", {
                "hidden": d, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": dh,
                "prefix": p + "self_attn.", "qk_norm": True, "eps": eps, "window": None,
                "position": PartSpec("rotate_half", {"head_dim": dh, "theta": cfg.rope_theta}),
            }),
            feed_forward_norm=PartSpec("rmsnorm", {"dim": d, "eps": eps, "name": p + "post_attention_layernorm.weight"}),
            feed_forward=PartSpec("swiglu", {"hidden": d, "inter": cfg.intermediate_size, "prefix": p + "mlp."}),
            arrangement="prenorm",
        ))
    return ModelSpec(
        architecture=cfg.ARCHITECTURE,
        vocab_size=cfg.vocab_size,
        hidden_size=d,
        embedding=PartSpec("table", {"vocab": cfg.vocab_size, "dim": d, "name": "model.embed_tokens.weight"}),
        layers=tuple(layers),
        schedule=tuple(Run(layer=i, cache=i) for i in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", {"dim": d, "eps": eps, "name": "model.norm.weight"}),
        head=PartSpec("linear", {"vocab": cfg.vocab_size, "dim": d, "name": "lm_head.weight",
                                 "tied": cfg.tie_word_embeddings}),
        max_positions=cfg.max_position_embeddings,
    )


register_architecture("Qwen3ForCausalLM", Qwen3Config, qwen3_spec, model_types=("qwen3",))
