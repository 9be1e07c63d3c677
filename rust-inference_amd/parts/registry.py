"""Registries of part kinds, one per category.

A new mixer, feed-forward, norm, position encoding or arrangement is a class
registered here under a name; a ``PartSpec`` of that name then builds it.  Tests
register toy parts the same way without touching the package.
"""
from __future__ import annotations

from ..errors import UnsupportedError

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "arrangement", "embedding", "head")
_REGISTRY: dict[str, dict[str, type]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, cls: type | None = None):
    """``register_part("mixer", "my_mixer", MyMixer)`` or as a class decorator."""
    if category not in _REGISTRY:
        raise UnsupportedError(f"no part category {category!r}; categories: {', '.join(CATEGORIES)}")

    def put(c):
        _REGISTRY[category][kind] = c
        return c

    return put(cls) if cls is not None else put


def part_class(category: str, kind: str) -> type:
    try:
        return _REGISTRY[category][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRY.get(category, {}))) or "none"
        raise UnsupportedError(f"no {category} part of kind {kind!r}; registered: {known}") from None


def build_part(category: str, spec, **extra):
    """An instance of the part a ``PartSpec`` names, with the spec's parameters."""
    return part_class(category, spec.kind)(**spec.params, **extra)


def registered(category: str) -> list[str]:
    return sorted(_REGISTRY[category])
