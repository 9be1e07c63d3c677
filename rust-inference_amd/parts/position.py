"""Position encodings."""
from __future__ import annotations

import torch

from ..errors import ConfigError
from .base import PositionEncoding
from .registry import register_part


@register_part("position", "rotate_half")
class RotateHalf(PositionEncoding):
    """Rotary encoding of the "default" kind over the whole head, pairs ``(d, d + dh/2)``.
    ``inv_freq[i] = 1 / theta^(2i / dh)`` in float32 (the reference: src/ops/rope.rs:20);
    the kernel forms the angle ``f32(pos) * inv_freq[i]`` in float32 (:39) and rotates
    ``x'[d] = x[d] cos - x[d+half] sin``, ``x'[d+half] = x[d+half] cos + x[d] sin`` (:73-74)."""

    def __init__(self, head_dim: int, theta: float):
        if head_dim % 2:
            raise ConfigError(f"head_dim {head_dim} must be even for a rotation in pairs")
        self.head_dim, self.theta = head_dim, theta

    def bind(self, weights, rt):
        self.rt = rt
        i = torch.arange(self.head_dim // 2, dtype=torch.float32)
        expo = (2.0 * i) / torch.tensor(float(self.head_dim), dtype=torch.float32)
        theta = torch.tensor(self.theta, dtype=torch.float32)
        self.inv_freq = (1.0 / torch.pow(theta, expo)).to(torch.float32).to(rt.device).contiguous()

    def bind_plain(self, weights):
        from ..kernels import plain
        self.inv_freq_plain = plain.rope_inv_freq(self.head_dim, self.theta)

    def plain(self, heads, positions):
        """Rotates ``heads: [tokens, n, head_dim]`` (already normed) by their tokens' positions."""
        from ..kernels import plain
        return plain.rope(heads, positions, self.inv_freq_plain)

    def rotation_table(self):
        return self.inv_freq


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position enters the mixer (order then comes from the causal mask alone)."""

    def __init__(self, **_):
        pass

    def bind_plain(self, weights):
        pass

    def plain(self, heads, positions):
        return heads
