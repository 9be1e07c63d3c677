"""A pool of fixed-size pages and each slot's table of them.

Pages are handed out lazily as a sequence grows, lowest number first, and go back
to the pool when the slot is released (the reference hands out page 0 first and
can only reset the whole cache: src/kvcache.rs:51, :115-124, :192-196).  A pool with
a window gives pages back as soon as every position in them lies behind the window
of all later queries.  The bookkeeping is native (csrc/host_cache.hip); ``tables`` is
a view of its memory.
"""
from __future__ import annotations

import numpy as np

from ..errors import CacheError
from . import native

UNMAPPED = -1


class PagePool:
    def __init__(self, num_pages: int, page_size: int, num_slots: int, max_pages_per_slot: int,
                 window: int | None = None):
        if page_size < 1 or num_pages < 1 or max_pages_per_slot < 1 or num_slots < 1:
            raise CacheError("page pool sizes must be positive")
        self.num_pages, self.page_size = num_pages, page_size
        self.max_pages_per_slot, self.window = max_pages_per_slot, window
        self._lib = native.lib()
        self.handle = self._lib.ri_pool_new(num_pages, page_size, num_slots, max_pages_per_slot, int(window or 0))
        if not self.handle:
            raise native.fail()
        # slot -> its pages by logical number, -1 where none is mapped: the pool's own memory
        self.tables = np.ctypeslib.as_array(self._lib.ri_pool_tables(self.handle), shape=(num_slots, max_pages_per_slot))

    def __del__(self):
        if getattr(self, "handle", None):
            self.tables = None
            self._lib.ri_pool_delete(self.handle)
            self.handle = None

    @property
    def free_count(self) -> int:
        return self._lib.ri_pool_free_count(self.handle)

    @property
    def capacity_per_slot(self) -> int:
        return self.max_pages_per_slot * self.page_size

    def pages_needed(self, slot: int, length_before: int, new_tokens: int) -> int:
        """How many pages ``reserve`` would take from the pool."""
        return self._lib.ri_pool_pages_needed(self.handle, int(slot), int(length_before), int(new_tokens))

    def reserve(self, slot: int, length_before: int, new_tokens: int) -> None:
        """Map pages for positions ``length_before .. length_before + new_tokens - 1``."""
        native.check(self._lib.ri_pool_reserve(self.handle, int(slot), int(length_before), int(new_tokens)))

    def trim_behind_window(self, slot: int, length: int) -> None:
        """Give back the pages that no query at a position >= ``length`` can see."""
        native.check(self._lib.ri_pool_trim(self.handle, int(slot), int(length)))

    def release(self, slot: int) -> None:
        native.check(self._lib.ri_pool_release(self.handle, int(slot)))

    def pages_of(self, slot: int) -> list[int]:
        row = self.tables[slot]
        return row[row != UNMAPPED].tolist()

    def gather(self, slots, width: int) -> np.ndarray:
        """The tables of these slots, ``[len(slots), width]``, unmapped places as -1."""
        return self.tables[np.asarray(slots, dtype=np.int64), :width]

    def check_consistent(self) -> None:
        """Every page is either free or in exactly one table; used by the tests."""
        native.check(self._lib.ri_pool_check(self.handle))
