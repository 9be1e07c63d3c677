"""A model as data: which parts each layer is made of and in which order layers run.

An architecture's builder turns its typed configuration into a ``ModelSpec``; the
generic ``DecoderModel`` is built from that.  Nothing here knows an architecture.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: its kind (a name in the part registry of its category) and its
    sizes, constants and tensor names as parameters."""
    kind: str
    params: dict = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement (how norms, mixer, feed-forward and the residual
    stream are wired) and the four parts it wires."""
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    arrangement: str = "prenorm"


@dataclass(frozen=True)
class Run:
    """One entry of the schedule: run layer ``layer`` with cache entry ``cache``.
    A layer may appear in several runs (its weights are shared, each run has its
    own cache entry), and two runs may name the same cache entry (the later one
    reads what the earlier one wrote; its mixer must be one that does not write)."""
    layer: int
    cache: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: tuple
    schedule: tuple
    final_norm: PartSpec
    head: PartSpec
    max_positions: int

    @property
    def num_cache_entries(self) -> int:
        used = [r.cache for r in self.schedule if r.cache is not None]
        return max(used) + 1 if used else 0
