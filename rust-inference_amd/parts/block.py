"""Arrangements: how a layer wires its norms, mixer and feed-forward around the residual stream."""
from __future__ import annotations

from .registry import build_part, register_part


class ResidualStream:
    """The float32 sum that runs through the layers, with at most one branch output
    waiting to be added.  The add is done by the next norm, in the same kernel."""

    def __init__(self, hidden):
        self.sum = hidden            # [T, hidden] float32
        self.pending = None

    def push(self, branch) -> None:
        if self.pending is not None:
            self.flush()
        self.pending = branch

    def normed(self, norm, out_dtype, rows=None):
        if self.pending is not None and self.pending.dim() == 3 and not getattr(norm, "accepts_parts", False):
            self.pending = self.pending.sum(0)       # a norm that does not know about parts
        out = norm.apply(self.sum, self.pending, out_dtype, rows)
        if rows is None:
            self.pending = None      # the kernel wrote sum + pending back
        return out

    def flush(self) -> None:
        """Add the waiting branch without a norm (only arrangements that push twice need it)."""
        if self.pending is not None:
            pending = self.pending.sum(0) if self.pending.dim() == 3 else self.pending
            self.sum.add_(pending.to(self.sum.dtype))
            self.pending = None


@register_part("arrangement", "prenorm")
class PreNormBlock:
    """``r = h + mixer(norm1(h))``, then ``h' = r + ff(norm2(r))``: the norm sits before
    each branch and the branch's output is added to the stream
    (the reference: src/models/qwen3.rs:121-145)."""

    def __init__(self, layer_spec):
        self.mixer_norm = build_part("norm", layer_spec.mixer_norm)
        self.mixer = build_part("mixer", layer_spec.mixer)
        self.feed_forward_norm = build_part("norm", layer_spec.feed_forward_norm)
        self.feed_forward = build_part("feed_forward", layer_spec.feed_forward)

    def parts(self):
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def forward(self, stream: ResidualStream, ctx, store, page_table, act_dtype) -> None:
        h = stream.normed(self.mixer_norm, act_dtype)
        stream.push(self.mixer.forward(h, ctx, store, page_table))
        h = stream.normed(self.feed_forward_norm, act_dtype)
        stream.push(self.feed_forward.forward(h, ctx))
