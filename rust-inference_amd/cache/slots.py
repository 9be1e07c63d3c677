"""Slots: one per live sequence of a batch.

A slot is the sequence's handle into every store of the cache (its row of each
page table, its row of each state arena).  It is acquired when the sequence
starts and released when it ends; a released slot is handed out again, lowest
number first.  The bookkeeping is native (csrc/host_cache.hip); a ``SlotAllocator``
made by itself has a core of its own, the cache's shares the cache's.
"""
from __future__ import annotations

from ..errors import CacheError
from . import native


class _Core:
    """Owner of a native cache core (slots, lengths, and the pools it was given)."""

    def __init__(self, pools, num_slots: int, max_seq_len: int):
        if num_slots < 1:
            raise CacheError("a cache needs at least one slot")
        lib = self._lib = native.lib()
        handles = (native.c_void_p * max(1, len(pools)))(*[p.handle for p in pools])
        self.pools = list(pools)                       # the core points into them: keep them alive
        self.handle = lib.ri_cache_new(handles, len(pools), num_slots, max_seq_len)
        if not self.handle:
            raise native.fail()

    def __del__(self):
        if getattr(self, "handle", None):
            self._lib.ri_cache_delete(self.handle)
            self.handle = None


class SlotAllocator:
    def __init__(self, num_slots: int, core: _Core | None = None):
        self.num_slots = num_slots
        self._core = core or _Core([], num_slots, 1)
        self._lib = native.lib()

    def acquire(self) -> int:
        slot = self._lib.ri_cache_acquire(self._core.handle)
        if slot < 0:
            raise native.fail()
        return slot

    def release(self, slot: int) -> None:
        native.check(self._lib.ri_cache_release(self._core.handle, int(slot)))

    def is_held(self, slot: int) -> bool:
        return bool(self._lib.ri_cache_is_held(self._core.handle, int(slot)))

    @property
    def free_count(self) -> int:
        return self._lib.ri_cache_free_slots(self._core.handle)
