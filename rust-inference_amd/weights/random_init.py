"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a seed.

Linear and embedding weights are N(0, 0.02) and norm gains 1 + N(0, 0.1), stored as
bfloat16 by default.  The reference's checkpoint script draws the same N(0, 0.02)
(scripts/synthetic_checkpoint.py:139-149) and its test builder the same gains
(scripts/reference_qwen3.py:216-217).  Every tensor has a generator of its own,
seeded from the seed and the tensor's name, so the values do not depend on the
order of creation and any one tensor can be made again alone.
"""
from __future__ import annotations

import hashlib
import json
import os

import torch

from ..config import config_from_dict
from .loader import GAIN, MATRIX, TABLE, TensorSpec
from .safetensors_io import save_file


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return g


def random_tensor(seed: int, name: str, spec: TensorSpec, dtype=torch.bfloat16, device="cpu",
                  matrix_std: float = 0.02, gain_std: float = 0.1) -> torch.Tensor:
    g = _generator(seed, name, device)
    if spec.kind == TABLE:
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    x = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
    if spec.kind == GAIN:
        x = 1.0 + gain_std * x
    else:
        x = matrix_std * x
    return x.to(dtype)


def random_tensors(expected: dict, seed: int, dtype=torch.bfloat16, device="cpu", **stds) -> dict:
    """One random tensor for every expected name (optional ones included unless the
    caller removed them from ``expected``)."""
    return {name: random_tensor(seed, name, spec, dtype, device, **stds) for name, spec in expected.items()}


def write_random_model(model_dir: str, config, seed: int, dtype=torch.bfloat16, **stds) -> str:
    """Make ``model_dir`` with config.json and model.safetensors for a configuration
    (a typed one or a config.json dict).  Returns the folder."""
    from ..parts.model import expected_tensors   # late: parts import the loader's kinds

    raw = config if isinstance(config, dict) else config.to_dict()
    arch, typed = config_from_dict(raw)
    spec = arch.build_spec(typed)
    expected = expected_tensors(spec, for_writing=True)
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        out = dict(raw)
        out.setdefault("architectures", [arch.name])
        out["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
        json.dump(out, f, indent=1)
    save_file(random_tensors(expected, seed, dtype, **stds), os.path.join(model_dir, "model.safetensors"),
              metadata={"format": "pt", "seed": seed})
    return model_dir


__all__ = ["random_tensor", "random_tensors", "write_random_model", "MATRIX", "GAIN", "TABLE"]
