"""Slots: one per live sequence of a batch.

A slot is the sequence's handle into every store of the cache (its row of each
page table, its row of each state arena).  It is acquired when the sequence
starts and released when it ends; a released slot is handed out again.
"""
from __future__ import annotations

from ..errors import CacheError


class SlotAllocator:
    def __init__(self, num_slots: int):
        if num_slots < 1:
            raise CacheError("a cache needs at least one slot")
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))   # popped from the back: slot 0 first
        self._held = [False] * num_slots

    def acquire(self) -> int:
        if not self._free:
            raise CacheError(f"no free slot: all {self.num_slots} are held by live sequences")
        slot = self._free.pop()
        self._held[slot] = True
        return slot

    def release(self, slot: int) -> None:
        self.check_held(slot)
        self._held[slot] = False
        self._free.append(slot)

    def check_held(self, slot: int) -> None:
        if not (0 <= slot < self.num_slots):
            raise CacheError(f"slot {slot} does not exist (the cache has {self.num_slots})")
        if not self._held[slot]:
            raise CacheError(f"slot {slot} is not held (never acquired, or released already)")

    def is_held(self, slot: int) -> bool:
        return 0 <= slot < self.num_slots and self._held[slot]

    @property
    def free_count(self) -> int:
        return len(self._free)

    def held_slots(self) -> list[int]:
        return [s for s in range(self.num_slots) if self._held[s]]
