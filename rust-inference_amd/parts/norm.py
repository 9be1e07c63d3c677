"""RMSNorm, fused with the residual add that precedes it."""
from __future__ import annotations

import torch

from ..kernels import ops, plain
from ..weights.loader import GAIN, TensorSpec
from .base import Norm
from .registry import register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    """``y = x * (1 / sqrt(mean(x^2) + eps)) * w`` over the last axis, statistics in
    float32 (the reference: src/ops/norm.rs:7-32; fused with the add: :35-62)."""

    accepts_parts = True
    linkable = True          # gain, eps and dim are all a product needs to do this norm itself
    can_tile = True          # hands its rows on in the matrix cores' order when asked (up to 64 rows)

    def __init__(self, dim: int, eps: float, name: str):
        self.dim, self.eps, self.name = dim, eps, name

    def tensors(self):
        return {self.name: TensorSpec((self.dim,), GAIN)}

    def bind(self, weights, rt):
        self.rt = rt
        self.gain = rt.place_gain(weights[self.name])

    def bind_plain(self, weights):
        self.gain_plain = weights[self.name].to(torch.float32).numpy()

    def plain(self, x):
        return plain.rms_norm(x, self.gain_plain, self.eps)

    def apply(self, residual, pending, out_dtype, rows=None, tiled=False):
        tiled = tiled and self.dim % 4 == 0 and self.dim <= 8192        # what the vectorised kernel takes
        return ops.add_rmsnorm(residual, pending, self.gain, self.eps, out_dtype, rows, tiled=tiled)
