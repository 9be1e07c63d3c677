"""Shared test set-up: the `gpu` marker, the two tiny configurations, model folders in temporary places."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # A test that hangs (a kernel whose waves never finish) should end the run and name itself rather than hold
    # the machine: where the timeout plugin is installed and the command line sets no limit, twenty minutes a test
    # (the longest, the kernels built for the CPU at a first call, takes five), ended from a watching thread (a
    # signal cannot interrupt a test that is stuck inside a GPU call).
    if config.pluginmanager.hasplugin("timeout") and not getattr(config.option, "timeout", None):
        config.option.timeout = 1200
        if not getattr(config.option, "timeout_method", None):
            config.option.timeout_method = "thread"


# Two tiny configurations of the architecture that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "vocab_size": 256, "hidden_size": 64, "intermediate_size": 128, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 128,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "vocab_size": 320, "hidden_size": 96, "intermediate_size": 160, "num_hidden_layers": 3,
    "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 32,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 256,
}
# A third one for long contexts and odd sizes: width and vocabulary that are no power of two,
# three query heads per kv head, head_dim 48.
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "vocab_size": 411, "hidden_size": 104, "intermediate_size": 232, "num_hidden_layers": 2,
    "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 48,
    "rope_theta": 50000.0, "rms_norm_eps": 3e-6, "tie_word_embeddings": False, "max_position_embeddings": 1024,
}
# The head size and grouping of the large models (128, four query heads per kv head), where the
# bfloat16 path takes its matrix-core attention kernels and packed weights.
TINY_D = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "vocab_size": 500, "hidden_size": 128, "intermediate_size": 384, "num_hidden_layers": 2,
    "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 128,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 512,
}


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders with random weights for the tiny configurations, made once per session.
    A is stored in float32, the others in bfloat16.  Weights are larger than the benchmark's
    N(0, 0.02) so that logits are of order one and differences show."""
    import torch
    from rust_inference_amd.weights import write_random_model
    base = tmp_path_factory.mktemp("models")
    out = {}
    for name, cfg, seed, dtype in (("A", TINY_A, 0, torch.float32), ("B", TINY_B, 1, torch.bfloat16),
                                   ("C", TINY_C, 2, torch.bfloat16), ("D", TINY_D, 3, torch.bfloat16)):
        out[name] = write_random_model(str(base / name), cfg, seed, dtype, matrix_std=0.12, gain_std=0.1)
    return out
