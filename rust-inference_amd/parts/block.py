"""Arrangements: how a layer wires its norms, mixer and feed-forward around the residual stream."""
from __future__ import annotations

import torch

from .. import profiler
from ..kernels import ops
from .registry import build_part, register_part

# A decode step of at most this many tokens leaves its norms to the products around them (the
# products that can do it take no more rows).
# (Links for the products of 17 to 32 rows were tried: with the sums of squares and the residual fetched at
# the end of the stream they cost what the two norm kernels cost at Qwen3-8B sizes, and 6% of the step at
# Qwen3-0.6B sizes.)
LINK_MAX_TOKENS = 16
# Up to this many rows a norm hands its rows on in the matrix cores' order when the reader asks.
TILED_MAX_ROWS = 64


class NormLink:
    """An offer to a branch's last product: add your result into ``residual`` yourself and prepare
    the rows for ``norm``, which then needs no kernel of its own."""

    def __init__(self, residual, norm, tiled: bool = False):
        self.residual, self.norm = residual, norm
        self.gain, self.eps = norm.gain, norm.eps
        self.tiled = tiled           # the reader of the prepared rows takes them in the matrix cores' order


class ResidualStream:
    """The float32 sum that runs through the layers, with at most one branch output
    waiting to be added.  The add is done by the next norm, in the same kernel, or, in
    small decode steps, by the product that made the branch output: then what waits is
    the prepared input of one norm (``later``) and the sum is already up to date."""

    def __init__(self, hidden):
        self.sum = hidden            # [T, hidden] float32
        self.pending = None
        self.later = None            # (NormedLater, the norm it was prepared for)
        self.next_entry_norm = None  # the norm that reads the stream after the current layer, if known
        self.next_entry_tiled = False  # and whether the part behind it reads tiled rows
        self.links_ok = True         # whether norms may be left to products at all (not where every step must run alike)

    def link(self, norm, act_dtype, tiled: bool = False):
        """A ``NormLink`` for the branch that is about to run, if ``norm`` is the next reader of the
        stream and can be left to a product.  ``tiled``: the part behind that norm reads tiled rows."""
        if (not self.links_ok or norm is None or not getattr(norm, "linkable", False) or self.pending is not None or self.later is not None
                or act_dtype != torch.bfloat16 or self.sum.shape[0] > LINK_MAX_TOKENS
                or norm.dim != self.sum.shape[1]):
            return None
        return NormLink(self.sum, norm, tiled)

    def push(self, branch) -> None:
        if self.pending is not None or self.later is not None:
            self.flush()
        if isinstance(branch, tuple):        # (NormedLater, norm): the product took a NormLink
            self.later = branch
        else:
            self.pending = branch

    def normed(self, norm, out_dtype, rows=None, later_ok: bool = False, tiled: bool = False):
        """The stream through ``norm``.  With ``later_ok`` the caller takes a ``NormedLater`` too, with
        ``tiled`` (a norm that can, up to 64 rows) ``ops.TiledRows``."""
        if self.later is not None:
            later, for_norm = self.later
            self.later = None
            if later_ok and for_norm is norm and rows is None:
                return later
            # prepared for another reader: the sum is complete, norm it the plain way
        if self.pending is not None and self.pending.dim() == 3 and not getattr(norm, "accepts_parts", False):
            self.flush()                             # a norm that does not know about parts: they go into the sum first
        with profiler.section(profiler.NORM):
            if (tiled and rows is None and getattr(norm, "can_tile", False) and out_dtype == torch.bfloat16
                    and self.sum.shape[0] <= TILED_MAX_ROWS):
                out = norm.apply(self.sum, self.pending, out_dtype, rows, tiled=True)
            else:
                out = norm.apply(self.sum, self.pending, out_dtype, rows)
        if rows is None:
            self.pending = None      # the kernel wrote sum + pending back
        return out

    def flush(self) -> None:
        """Add the waiting branch without a norm (only arrangements that push twice need it)."""
        self.later = None            # its sum is in the stream already
        if self.pending is not None:
            for part in (self.pending.unbind(0) if self.pending.dim() == 3 else (self.pending,)):
                ops.add_rows(self.sum, part, in_place=True)       # parts in order, each sum in float32
            self.pending = None


def _takes_tiled(part, rows: int) -> bool:
    asks = getattr(part, "takes_tiled_at", None)
    return bool(asks(rows)) if asks else False


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

    def entry_norm(self):
        """The norm through which this layer first reads the stream."""
        return self.mixer_norm

    def entry_takes_tiled(self, rows: int) -> bool:
        """Whether the part behind that norm reads ``rows`` rows in the matrix cores' order."""
        return _takes_tiled(self.mixer, rows)

    def plain(self, h, ctx, store, page_table):
        """``h`` after this layer, float32 numpy (the plain backend)."""
        r = h + self.mixer.plain(self.mixer_norm.plain(h), ctx, store, page_table)
        return r + self.feed_forward.plain(self.feed_forward_norm.plain(r), ctx)

    def forward(self, stream: ResidualStream, ctx, store, page_table, act_dtype) -> None:
        # a part with ``links_norms`` takes a NormedLater as input and a NormLink for its output
        rows = stream.sum.shape[0]
        if getattr(self.mixer, "links_norms", False):
            h = stream.normed(self.mixer_norm, act_dtype, later_ok=True, tiled=_takes_tiled(self.mixer, rows))
            link = stream.link(self.feed_forward_norm, act_dtype, _takes_tiled(self.feed_forward, rows))
            stream.push(self.mixer.forward(h, ctx, store, page_table, link=link))
        else:
            h = stream.normed(self.mixer_norm, act_dtype)
            stream.push(self.mixer.forward(h, ctx, store, page_table))
        if getattr(self.feed_forward, "links_norms", False):
            h = stream.normed(self.feed_forward_norm, act_dtype, later_ok=True,
                              tiled=_takes_tiled(self.feed_forward, rows))
            link = stream.link(stream.next_entry_norm, act_dtype, stream.next_entry_tiled)
            stream.push(self.feed_forward.forward(h, ctx, link=link))
        else:
            h = stream.normed(self.feed_forward_norm, act_dtype)
            stream.push(self.feed_forward.forward(h, ctx))
