"""Configuration and registry (no GPU)."""
import json

import pytest

from conftest import TINY_A, TINY_B
from rust_inference_amd.config import Qwen3Config, config_from_dict, known_architectures, load_config
from rust_inference_amd.errors import ConfigError, UnsupportedError
from rust_inference_amd.parts import expected_tensors
from rust_inference_amd.parts.qwen3 import qwen3_spec


def minimal():
    return {"architectures": ["Qwen3ForCausalLM"], "vocab_size": 10, "hidden_size": 8, "intermediate_size": 16,
            "num_hidden_layers": 4, "num_attention_heads": 2, "num_key_value_heads": 1}


def test_defaults_follow_the_reference():
    # src/models/config.rs:57-65, :35-36, :75-77
    _, c = config_from_dict(minimal())
    assert c.dim_per_head == 4 and c.max_position_embeddings == 40960 and c.tie_word_embeddings is False
    assert abs(c.rms_norm_eps - 1e-6) < 1e-12 and c.rope_theta == 1e6


def test_eps_and_theta_are_32_bit_numbers():
    raw = dict(minimal(), rms_norm_eps=1e-6, rope_theta=1234567.891)
    _, c = config_from_dict(raw)
    import numpy as np
    assert c.rms_norm_eps == float(np.float32(1e-6)) and c.rope_theta == float(np.float32(1234567.891))


def test_head_dim_is_its_own_key():
    _, c = config_from_dict(dict(minimal(), head_dim=16))
    assert c.dim_per_head == 16          # heads * head_dim != hidden is legal


def test_model_type_selects_when_architectures_is_absent():
    raw = minimal()
    del raw["architectures"]
    raw["model_type"] = "qwen3"
    arch, _ = config_from_dict(raw)
    assert arch.name == "Qwen3ForCausalLM"


@pytest.mark.parametrize("patch, error", [
    ({"num_attention_heads": 3}, ConfigError),                                # not divisible by kv heads... 3 % 1 ok -> head_dim
    ({"num_key_value_heads": 0}, ConfigError),
    ({"num_attention_heads": 4, "num_key_value_heads": 3}, ConfigError),
    ({"head_dim": 7}, ConfigError),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 4.0}}, ConfigError),    # src/models/config.rs:104-109
    ({"num_experts": 4}, UnsupportedError),
    ({"quantization_config": {"quant_method": "fp8"}}, UnsupportedError),
    ({"architectures": ["LlamaForCausalLM"]}, UnsupportedError),
    ({"vocab_size": "many"}, ConfigError),
])
def test_refused_configurations(patch, error):
    with pytest.raises(error):
        config_from_dict(dict(minimal(), **patch))


def test_default_rope_scaling_is_accepted():
    config_from_dict(dict(minimal(), rope_scaling={"rope_type": "default"}))
    config_from_dict(dict(minimal(), rope_scaling=None))


def test_missing_keys_are_named():
    raw = minimal()
    del raw["intermediate_size"], raw["vocab_size"]
    with pytest.raises(ConfigError, match="vocab_size.*intermediate_size|intermediate_size.*vocab_size"):
        config_from_dict(raw)


def test_unknown_architecture_lists_the_known_ones():
    with pytest.raises(UnsupportedError, match="Qwen3ForCausalLM"):
        config_from_dict({"architectures": ["Nope"]})
    assert "Qwen3ForCausalLM" in known_architectures()


def test_load_config_reads_a_folder_and_names_the_path(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, c = load_config(str(tmp_path))
    assert isinstance(c, Qwen3Config) and c.num_hidden_layers == 3 and c.rms_norm_eps == pytest.approx(1e-5)
    assert config_from_dict(c.to_dict())[1] == c          # the written config reads back the same


def test_every_size_of_the_spec_comes_from_the_configuration():
    for raw in (TINY_A, TINY_B):
        _, c = config_from_dict(raw)
        spec = qwen3_spec(c)
        t = expected_tensors(spec)
        d, dh, h, hkv, i, v = (c.hidden_size, c.dim_per_head, c.num_attention_heads, c.num_key_value_heads,
                               c.intermediate_size, c.vocab_size)
        assert t["model.embed_tokens.weight"].shape == (v, d)
        assert t["model.layers.0.self_attn.q_proj.weight"].shape == (h * dh, d)
        assert t["model.layers.0.self_attn.k_proj.weight"].shape == (hkv * dh, d)
        assert t["model.layers.0.self_attn.o_proj.weight"].shape == (d, h * dh)
        assert t["model.layers.0.self_attn.q_norm.weight"].shape == (dh,)
        assert t["model.layers.0.mlp.down_proj.weight"].shape == (d, i)
        assert t["lm_head.weight"].optional
        assert len(spec.layers) == c.num_hidden_layers == len(spec.schedule)
        assert len(t) == 3 + 11 * c.num_hidden_layers
        mixer = spec.layers[0].mixer.params
        assert mixer["eps"] == c.rms_norm_eps and mixer["position"].params["theta"] == c.rope_theta
