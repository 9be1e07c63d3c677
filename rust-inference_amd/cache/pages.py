"""A pool of fixed-size pages and each slot's table of them.

Pages are handed out lazily as a sequence grows, lowest number first, and go back
to the pool when the slot is released (the reference hands out page 0 first and
can only reset the whole cache: src/kvcache.rs:51, :115-124, :192-196).  A pool with
a window gives pages back as soon as every position in them lies behind the window
of all later queries.
"""
from __future__ import annotations

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
        self.tables = [[UNMAPPED] * max_pages_per_slot for _ in range(num_slots)]

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def capacity_per_slot(self) -> int:
        return self.max_pages_per_slot * self.page_size

    def pages_needed(self, slot: int, length_before: int, new_tokens: int) -> int:
        """How many pages ``reserve`` would take from the pool."""
        table = self.tables[slot]
        first, last = length_before // self.page_size, -(-(length_before + new_tokens) // self.page_size)
        return sum(1 for p in range(first, min(last, self.max_pages_per_slot)) if table[p] == UNMAPPED)

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
                table[logical] = page

    def _give_back(self, slot: int, logical: int) -> None:
        page = self.tables[slot][logical]
        if page == UNMAPPED:
            return
        if self._owner[page] != slot:
            raise CacheError(f"page {page} is in slot {slot}'s table but owned by {self._owner[page]}")
        self._owner[page] = UNMAPPED
        self.tables[slot][logical] = UNMAPPED
        self._free.append(page)

    def trim_behind_window(self, slot: int, length: int) -> None:
        """Give back the pages that no query at a position >= ``length`` can see."""
        if self.window is None:
            return
        first_visible = max(0, length - self.window + 1)     # of the next query, at position `length`
        for logical in range(0, first_visible // self.page_size):
            self._give_back(slot, logical)

    def release(self, slot: int) -> None:
        for logical in range(self.max_pages_per_slot):
            self._give_back(slot, logical)

    def pages_of(self, slot: int) -> list[int]:
        return [p for p in self.tables[slot] if p != UNMAPPED]

    def check_consistent(self) -> None:
        """Every page is either free or in exactly one table; used by the tests."""
        seen = {}
        for slot, table in enumerate(self.tables):
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
