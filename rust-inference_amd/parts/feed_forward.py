"""Feed-forward parts."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import MATRIX, TensorSpec
from .base import FeedForward
from .registry import register_part
from .runtime import GEMV_MAX_ROWS


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))``, no bias, ``silu(z) = z / (1 + exp(-z))``
    (the reference: src/models/qwen3.rs:112-117; src/ops/elementwise.rs:9-12).  Gate and
    up are one product with the row-concatenated weight ``[gate; up]``."""

    def __init__(self, hidden: int, inter: int, prefix: str):
        self.hidden, self.inter, self.prefix = hidden, inter, prefix

    def tensors(self):
        p = self.prefix
        return {
            p + "gate_proj.weight": TensorSpec((self.inter, self.hidden), MATRIX),
            p + "up_proj.weight": TensorSpec((self.inter, self.hidden), MATRIX),
            p + "down_proj.weight": TensorSpec((self.hidden, self.inter), MATRIX),
        }

    def bind(self, weights, rt):
        self.rt = rt
        p = self.prefix
        self.w_gate_up = rt.place_matrix(torch.cat([weights[p + "gate_proj.weight"], weights[p + "up_proj.weight"]], 0))
        self.w_down = rt.place_matrix(weights[p + "down_proj.weight"])

    def forward(self, x, ctx):
        rt = self.rt
        if rt.dtype == torch.bfloat16 and x.shape[0] <= GEMV_MAX_ROWS and self.hidden % 8 == 0:
            a = ops.gemv_bf16(x, self.w_gate_up, torch.bfloat16, swiglu=True)      # activation in the epilogue
        else:
            a = ops.swiglu(rt.linear(x, self.w_gate_up))
        return rt.linear(a, self.w_down)
