"""A pool of fixed-size pages and each slot's table of them.

Pages are handed out lazily as a sequence grows, lowest number first, and go back
to the pool when the slot is released (the reference hands out page 0 first and
can only reset the whole cache: src/kvcache.rs:51, :115-124, :192-196).  A pool with
a window gives pages back as soon as every position in them lies behind the window
of all later queries.
"""
from __future__ import annotations

import numpy as np

from ..errors import CacheError

UNMAPPED = -1


class PagePool:
    def __init__(self, num_pages: int, page_size: int, num_slots: int, max_pages_per_slot: int,
                 window: int | None = None):
        if page_size < 1 or num_pages < 1 or max_pages_per_slot < 1:
            raise CacheError("page pool sizes must be positive")
        self.num_pages, self.page_size = num_pages, page_size
        self.max_pages_per_slot, self.window = max_pages_per_slot, window
        self._free = list(range(num_pages - 1, -1, -1))
        self._owner = [UNMAPPED] * num_pages             # page -> slot, to catch double frees
        # slot -> its pages by logical number: one array, so that a step's tables are one gather
        self.tables = np.full((num_slots, max_pages_per_slot), UNMAPPED, dtype=np.int32)

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def capacity_per_slot(self) -> int:
        return self.max_pages_per_slot * self.page_size

    def pages_needed(self, slot: int, length_before: int, new_tokens: int) -> int:
        """How many pages ``reserve`` would take from the pool."""
        first, last = length_before // self.page_size, -(-(length_before + new_tokens) // self.page_size)
        if last - first == 1 and last <= self.max_pages_per_slot:          # the usual step: one token more
            return int(self.tables[slot, first] == UNMAPPED)
        return int((self.tables[slot, first:min(last, self.max_pages_per_slot)] == UNMAPPED).sum())

    def reserve(self, slot: int, length_before: int, new_tokens: int) -> None:
        """Map pages for positions ``length_before .. length_before + new_tokens - 1``."""
        end = length_before + new_tokens
        if end > self.capacity_per_slot:
            raise CacheError(f"slot {slot} would reach {end} tokens, the cache holds {self.capacity_per_slot} "
                             f"per sequence")                                      # src/kvcache.rs:109-114
        table = self.tables[slot]
        for logical in range(length_before // self.page_size, -(-end // self.page_size)):
            if table[logical] == UNMAPPED:
                if not self._free:
                    raise CacheError(f"cache out of pages ({self.num_pages} of {self.page_size} tokens in all)")
                page = self._free.pop()
                self._owner[page] = slot
                table[logical] = page                                              # (a view: writes the array)

    def _give_back(self, slot: int, logical: int) -> None:
        page = int(self.tables[slot, logical])
        if page == UNMAPPED:
            return
        if self._owner[page] != slot:
            raise CacheError(f"page {page} is in slot {slot}'s table but owned by {self._owner[page]}")
        self._owner[page] = UNMAPPED
        self.tables[slot, logical] = UNMAPPED
        self._free.append(page)

    def trim_behind_window(self, slot: int, length: int) -> None:
        """Give back the pages that no query at a position >= ``length`` can see."""
        if self.window is None:
            return
        first_visible = max(0, length - self.window + 1)     # of the next query, at position `length`
        for logical in range(0, first_visible // self.page_size):
            self._give_back(slot, logical)

    def release(self, slot: int) -> None:
        for logical in np.nonzero(self.tables[slot] != UNMAPPED)[0].tolist():
            self._give_back(slot, logical)

    def pages_of(self, slot: int) -> list[int]:
        row = self.tables[slot]
        return row[row != UNMAPPED].tolist()

    def gather(self, slots, width: int) -> np.ndarray:
        """The tables of these slots, ``[len(slots), width]``, unmapped places as -1."""
        return self.tables[np.asarray(slots, dtype=np.int64), :width]

    def check_consistent(self) -> None:
        """Every page is either free or in exactly one table; used by the tests."""
        seen = {}
        for slot, table in enumerate(self.tables.tolist()):
            for page in table:
                if page == UNMAPPED:
                    continue
                if page in seen:
                    raise CacheError(f"page {page} is held twice (slots {seen[page]} and {slot})")
                seen[page] = slot
                if self._owner[page] != slot:
                    raise CacheError(f"page {page}: owner {self._owner[page]} but in slot {slot}'s table")
        free = set(self._free)
        if len(free) != len(self._free):
            raise CacheError("a page is on the free list twice")
        if free & set(seen):
            raise CacheError("a page is both free and held")
        if len(free) + len(seen) != self.num_pages:
            raise CacheError(f"{self.num_pages - len(free) - len(seen)} pages are lost")
