"""A model as data: which parts each layer is made of and in which order layers run.

An architecture's builder turns its typed configuration into a ``ModelSpec``; the
generic ``DecoderModel`` is built from that.  Nothing here knows an architecture.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from types import MappingProxyType
from typing import Mapping, Optional, Tuple, Union


@dataclass(frozen=True)
class PartSpec:
    """One part: its kind (a name in the part registry of its category) and its
    sizes, constants and tensor names as parameters."""
    kind: str
    params: dict = field(default_factory=dict)


class LayerSpec:
    """One layer: an arrangement (how norms, mixers, feed-forwards and the residual stream are wired) and
    the parts it wires, by name.  Which names there are is the arrangement's business: the pre-norm block
    reads ``mixer_norm``, ``mixer``, ``feed_forward_norm`` and ``feed_forward``; an arrangement with norms
    on both sides of a branch, with two mixers side by side or with no feed-forward at all names its own.

        LayerSpec(arrangement="prenorm", mixer=PartSpec(...), feed_forward=PartSpec(...), ...)
        LayerSpec("sandwich", parts={"mixer": ..., "mixer_norm": ..., "after_mixer_norm": ..., ...})

    A named part is read as an attribute (``spec.mixer``) or from ``spec.parts``."""

    def __init__(self, arrangement: str = "prenorm", parts: Optional[Mapping[str, PartSpec]] = None, **named: PartSpec):
        merged = dict(parts or {})
        merged.update(named)
        for name, part in merged.items():
            if not isinstance(part, PartSpec):
                raise TypeError(f"part {name!r} of a layer must be a PartSpec, not {type(part).__name__}")
        object.__setattr__(self, "arrangement", arrangement)
        object.__setattr__(self, "parts", MappingProxyType(merged))

    def __getattr__(self, name: str) -> PartSpec:
        try:
            return self.__dict__["parts"][name]
        except KeyError:
            raise AttributeError(f"this layer has no part named {name!r} (it has: {', '.join(self.__dict__.get('parts', {}))})") from None

    def __setattr__(self, name, value):
        raise AttributeError("a LayerSpec is not changed after it is made")

    def __eq__(self, other):
        return isinstance(other, LayerSpec) and (self.arrangement, dict(self.parts)) == (other.arrangement, dict(other.parts))

    def __repr__(self):
        return f"LayerSpec({self.arrangement!r}, {dict(self.parts)!r})"


@dataclass(frozen=True)
class Run:
    """One entry of the schedule: run layer ``layer`` with cache entry ``cache``.
    A layer may appear in several runs (its weights are shared, each run has its
    own cache entry), and two runs may name the same cache entry (the later one
    reads what the earlier one wrote; its mixer must be one that does not write).
    A layer that keeps more than one thing per sequence (keys and values and a state
    of fixed size, or the caches of two mixers) names a tuple of entries, one for each
    need its ``cache_need()`` lists, in that order."""
    layer: int
    cache: Union[None, int, Tuple[int, ...]] = None

    def entries(self) -> Tuple[int, ...]:
        if self.cache is None:
            return ()
        return (self.cache,) if isinstance(self.cache, int) else tuple(self.cache)


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
        used = [e for r in self.schedule for e in r.entries()]
        return max(used) + 1 if used else 0
