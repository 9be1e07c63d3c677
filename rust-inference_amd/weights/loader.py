"""Loading a model's tensors by name and checking them against what the model expects.

The model says which tensors it wants (name, shape, kind); the loader compares
that with the folder and raises ONE error that lists every missing tensor, every
wrong shape and dtype, and with them the tensors the model did not expect.  A folder
whose only oddity is tensors the model does not read loads, as it does in the
reference, which looks tensors up by name and never lists the rest
(src/safetensors.rs:157-174); they are named in one warning.  Tensors keep the dtype they are stored in:
bfloat16 stays bfloat16 and a tensor stored in 32-bit stays 32-bit; integer tables
become int32.
"""
from __future__ import annotations

import warnings
from dataclasses import dataclass

import torch

from ..errors import WeightsError
from .safetensors_io import ModelFolder

MATRIX = "matrix"     # linear and embedding weights: N(0, 0.02) when random
GAIN = "gain"         # norm gains: 1 + N(0, 0.1) when random; always used in 32-bit
TABLE = "table"       # integer tables
BIAS = "bias"         # biases of products: drawn like matrices when random, used in 32-bit like gains


@dataclass(frozen=True)
class TensorSpec:
    shape: tuple
    kind: str = MATRIX
    optional: bool = False     # absent is fine (e.g. lm_head.weight of a tied model)


_KEPT = (torch.bfloat16, torch.float32)


def check_folder(folder: ModelFolder, expected: dict[str, TensorSpec]) -> None:
    missing, unexpected, misshapen, wrong_dtype = [], [], [], []
    for name, spec in expected.items():
        if name not in folder:
            if not spec.optional:
                missing.append(name)
            continue
        info = folder.info(name)
        if tuple(info.shape) != tuple(spec.shape):
            misshapen.append(f"{name}: file has {list(info.shape)}, model wants {list(spec.shape)}")
        if info.dtype is None:
            wrong_dtype.append(f"{name}: stored as {info.stored_as}, which this library does not read")
        elif spec.kind == TABLE:
            if info.dtype not in (torch.int32, torch.int64):
                wrong_dtype.append(f"{name}: {info.dtype} is not an integer table")
        elif info.dtype not in _KEPT:
            wrong_dtype.append(f"{name}: {info.dtype} is neither bfloat16 nor float32")
    for name in folder.names():
        if name not in expected:
            unexpected.append(name)
    if unexpected and not (missing or misshapen or wrong_dtype):
        shown = ", ".join(unexpected[:8]) + (f" and {len(unexpected) - 8} more" if len(unexpected) > 8 else "")
        warnings.warn(f"{folder.model_dir}: {len(unexpected)} tensors that the model does not read are ignored: {shown}",
                      stacklevel=3)
        return
    if missing or misshapen or wrong_dtype:
        parts = []
        if missing:
            parts.append(f"missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            parts.append(f"unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if misshapen:
            parts.append(f"wrong shape ({len(misshapen)}): " + "; ".join(misshapen))
        if wrong_dtype:
            parts.append(f"wrong dtype ({len(wrong_dtype)}): " + "; ".join(wrong_dtype))
        raise WeightsError(f"{folder.model_dir} does not fit the model\n  " + "\n  ".join(parts))


def load_checked(model_dir: str, expected: dict[str, TensorSpec]) -> dict[str, torch.Tensor]:
    """All expected tensors that the folder has, as views of the mapped files."""
    folder = ModelFolder(model_dir)
    check_folder(folder, expected)
    out = {}
    for name, spec in expected.items():
        if name in folder:
            t = folder.load(name)
            out[name] = t.to(torch.int32) if spec.kind == TABLE else t
    return out
