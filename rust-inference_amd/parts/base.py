"""Interfaces of the parts.

Every part: is built from the parameters of its ``PartSpec``; says which tensors
it wants (``tensors()``: checkpoint name -> ``TensorSpec``); takes them over
(``bind(weights, runtime)``); and runs on the flattened tokens of a step.  No part
knows which model it is in.
"""
from __future__ import annotations

from ..weights.loader import TensorSpec


class Part:
    """A part may also run on the CPU, for the plain backend (engine/plain_engine.py: the whole model over the
    scalar C++ twins of the kernels, in float32, as the reference's CPU path computes: src/ops/mod.rs:36-41,
    src/cpu/linear.rs:119-130): ``bind_plain(weights)`` keeps what it needs as float32 numpy arrays and
    ``plain(...)`` is its forward over numpy arrays, with the arguments of ``forward`` (a mixer's store is the
    pair of page arrays ``(k_pages, v_pages)`` or its state arena).  A part without them cannot run there."""

    def tensors(self) -> dict[str, TensorSpec]:
        """Checkpoint names and shapes of this part's weights."""
        return {}

    def bind(self, weights: dict, rt) -> None:
        """Take the weights (host tensors, as stored) and put what is needed on the device."""
        self.rt = rt

    def connect(self, parts: dict) -> None:
        """Called once after every part of the model is bound, with the model's own parts by name
        (``"embedding"``, ``"final_norm"``, ``"head"``, ``"layers"``): for a part that shares something with
        another one (an output matrix tied to the embedding table).  Most parts need nothing here."""


class Embedding(Part):
    """``forward(ctx) -> [T, hidden]`` float32: what the residual stream starts from.  The part gets the whole
    step's context, so one that adds something by position (``ctx.tok_pos``) or by sequence (``ctx.tok_seq``,
    ``ctx.slots``) to the rows of its table needs nothing from the model."""

    def forward(self, ctx):
        raise NotImplementedError


class Head(Part):
    """``forward(x) -> [rows, vocab]`` float32 logits of the final norm's rows."""

    def forward(self, x):
        raise NotImplementedError


class Norm(Part):
    """``apply(residual, pending, out_dtype, rows=None)``: adds ``pending`` into the
    float32 residual stream (in place when ``rows`` is None) and returns the norm of
    the sum in ``out_dtype``; with ``rows`` only those rows, nothing written back.  A norm that sets
    ``accepts_parts`` also takes ``pending`` as ``[parts, T, hidden]`` and adds the parts in order."""

    accepts_parts = False

    def apply(self, residual, pending, out_dtype, rows=None):
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the tokens of a sequence.

    ``cache_need()`` says what one cache entry of this mixer holds (a ``KVNeed``, a
    ``StateNeed`` or None).  ``forward(x, ctx, store, page_table)`` gets the normed
    tokens ``[T, hidden]``, the step's context, its cache entry's storage (a
    ``KVView`` or the state arena ``[slots, ...]``) and, for key/value needs, the
    step's page table of its group; it returns ``[T, hidden]``.  Tokens of a
    sequence are contiguous and in order (``ctx.cu_seqlens``); a mixer with state
    reads its slot's row, consumes the sequence's tokens in order and writes the
    row back.  Decode steps may be captured as a graph and replayed for other slots
    and positions: a mixer that is to run there takes them from the context's device
    tensors (``ctx.slots``, ``ctx.tok_pos``, the page table), not from its host lists.
    """

    def cache_need(self):
        return None

    def forward(self, x, ctx, store, page_table):
        raise NotImplementedError


class FeedForward(Part):
    """Token-wise ``[T, hidden] -> [T, hidden]``.  The result may also be ``[parts, T, hidden]`` float32:
    partial sums that the residual stream adds up in order (a product split along K)."""

    def forward(self, x, ctx):
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter a mixer.  ``rotation_table()`` returns float32 inverse frequencies ``[r]``
    (``r <= head_dim / 2``) for the fused kernel, which rotates the first ``2 r`` elements of every q and k
    head in pairs ``(i, i + r)`` by ``pos * inv_freq[i]`` after the per-head norm, or None when this
    encoding does not rotate.  An encoding of another kind changes q and k itself, in place, in the fused
    projection ``qkv: [T, (heads + 2 kv_heads) * head_dim]``: in ``apply`` before the per-head norm, or,
    when it sets ``acts_after_norm``, in ``apply_normed`` after the norm (and after the rotation, if it
    also has a table) and before k and v go to the cache; the mixer then runs the norm, the encoding and
    the cache write as three steps instead of one kernel."""

    acts_after_norm = False

    def rotation_table(self):
        return None

    def apply(self, qkv, ctx, heads, kv_heads, head_dim):
        return None

    def apply_normed(self, qkv, ctx, heads, kv_heads, head_dim):
        return None
