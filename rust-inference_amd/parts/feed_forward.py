"""Feed-forward parts."""
from __future__ import annotations

import torch

from .. import profiler
from ..weights.loader import MATRIX, TensorSpec
from .base import FeedForward
from .registry import register_part


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))``, no bias, ``silu(z) = z / (1 + exp(-z))``
    (the reference: src/models/qwen3.rs:112-117; src/ops/elementwise.rs:9-12).  Gate and
    up are one product with the row-concatenated weight ``[gate; up]``."""

    links_norms = True

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
        gate_up = rt.place_matrix(torch.cat([weights[p + "gate_proj.weight"], weights[p + "up_proj.weight"]], 0))
        self.w_gate_up = rt.pack(gate_up, swiglu=True)
        self.w_down = rt.pack(rt.place_matrix(weights[p + "down_proj.weight"]), parts_ok=True)

    def bind_plain(self, weights):
        p = self.prefix
        self.plain_w = {n: weights[p + n + "_proj.weight"].to(torch.float32).numpy() for n in ("gate", "up", "down")}

    def plain(self, x, ctx):
        from ..kernels import plain
        import numpy as np
        y = np.concatenate([plain.linear(x, self.plain_w["gate"]), plain.linear(x, self.plain_w["up"])], axis=1)
        return plain.linear(plain.swiglu(y), self.plain_w["down"])

    def takes_tiled_at(self, m: int) -> bool:
        """Whether this part's first product reads ``m`` rows in the matrix cores' order."""
        return self.rt.takes_tiled(self.w_gate_up, m)

    def forward(self, x, ctx, link=None):
        rt = self.rt
        # the activation is in the epilogue of the decode-size kernels, which hand the down product its rows
        # in the order it loads fastest when that product is a packed one too
        with profiler.section(profiler.MLP):
            a = rt.linear_packed(x, self.w_gate_up, tiled_out=rt.takes_tiled(self.w_down, x.shape[0], True))
            # may come in parts: the stream's next norm adds them
            return rt.linear_packed(a, self.w_down, parts_ok=True, link=link)
