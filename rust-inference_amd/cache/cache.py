"""The cache: what live sequences keep between steps.

A model's mixers say what they need per cache entry: keys and values for every
token (optionally only a window of them), or a state of fixed size per sequence.
Entries with the same key/value geometry form a group with storage and a page
pool of its own; every state entry has an arena of its own, one row per slot.
A sequence holds one slot from its first step to its end, and the slot addresses
all of these.  Lengths are per slot: sequences of a batch advance by different
numbers of tokens.

The reference keeps one page table per layer and advances every sequence by the
same count (src/kvcache.rs:106-135, :185-187); here one table serves all layers
of a group and is sent to the device once per step.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

from ..errors import CacheError
from . import native
from .pages import PagePool, UNMAPPED
from .slots import SlotAllocator, _Core

PAGE_SIZE = 32   # tokens per page, as in the reference (src/kvcache.rs:12)


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of ``kv_heads`` heads of ``head_dim`` for every token, or for
    the last ``window`` tokens only."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """A tensor of fixed shape per sequence, zero when the sequence starts."""
    shape: tuple
    dtype: torch.dtype = torch.float32


class KVGroup:
    """Storage for all cache entries that share one key/value geometry.

    ``k_pages[e]`` is ``[num_pages, kv_heads, page_size, head_dim]`` for entry ``e`` of
    the group (the reference's layout: src/kvcache.rs:42-50, :145-147).  ``v_pages[e]`` is
    ``[num_pages, kv_heads, head_dim, page_size]``: values lie transposed inside a page,
    the page's tokens contiguous for each channel, because that is the operand order
    the matrix cores want for the product of weights and values.  One page number
    means the same page in every entry.
    """

    def __init__(self, need: KVNeed, entries: list[int], num_pages: int, num_slots: int,
                 max_pages_per_slot: int, page_size: int, dtype, device, allocate: bool):
        self.need, self.entries, self.page_size = need, list(entries), page_size
        self.pool = PagePool(num_pages, page_size, num_slots, max_pages_per_slot, need.window)
        self.index_of = {e: i for i, e in enumerate(self.entries)}
        k_shape = (len(self.entries), num_pages, need.kv_heads, page_size, need.head_dim)
        v_shape = (len(self.entries), num_pages, need.kv_heads, need.head_dim, page_size)
        self.k_pages = torch.zeros(k_shape, dtype=dtype, device=device) if allocate else None
        self.v_pages = torch.zeros(v_shape, dtype=dtype, device=device) if allocate else None


@dataclass
class KVView:
    """What a mixer gets for its cache entry in a step."""
    group_index: int
    k_pages: torch.Tensor
    v_pages: torch.Tensor
    page_size: int
    window: Optional[int]


class Cache:
    def __init__(self, needs: Sequence[object], num_slots: int, max_tokens: int, max_seq_len: int,
                 dtype=torch.bfloat16, device="cpu", page_size: int = PAGE_SIZE, allocate: bool = True):
        """``needs[e]`` is the need of cache entry ``e`` (None for an entry nothing
        uses).  ``max_tokens`` is the most tokens all live sequences hold together,
        each sequence's count rounded up to whole pages; ``max_seq_len`` is the most
        one sequence may hold."""
        if max_tokens < 1 or max_seq_len < 1:
            raise CacheError("max_tokens and max_seq_len must be positive")
        self.page_size, self.num_slots = page_size, num_slots
        self.max_seq_len = max_seq_len
        self.device, self.dtype = device, dtype
        self.max_pages_per_slot = -(-max_seq_len // page_size)
        num_pages = -(-max_tokens // page_size)
        self.needs = list(needs)
        self.groups: list[KVGroup] = []
        self._kv_of_entry: dict[int, tuple[int, int]] = {}
        self._state: dict[int, torch.Tensor] = {}
        by_need: dict[KVNeed, list[int]] = {}
        for e, need in enumerate(self.needs):
            if isinstance(need, KVNeed):
                by_need.setdefault(need, []).append(e)
            elif isinstance(need, StateNeed):
                self._state[e] = torch.zeros((num_slots, *need.shape), dtype=need.dtype, device=device)
            elif need is not None:
                raise CacheError(f"cache entry {e}: unknown need {need!r}")
        for need, entries in by_need.items():
            g = KVGroup(need, entries, num_pages, num_slots, self.max_pages_per_slot, page_size, dtype, device, allocate)
            for e in entries:
                self._kv_of_entry[e] = (len(self.groups), g.index_of[e])
            self.groups.append(g)
        # slots, lengths and the groups' pools together: native bookkeeping (csrc/host_cache.hip)
        self.core = _Core([g.pool for g in self.groups], num_slots, max_seq_len)
        self.slots = SlotAllocator(num_slots, self.core)
        self._lib = native.lib()

    # ---- slots
    def acquire(self) -> int:
        slot = self.slots.acquire()                 # comes back with length 0
        for arena in self._state.values():
            arena[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        self.slots.release(slot)                    # its pages go back to every pool, its length to 0

    def length(self, slot: int) -> int:
        n = self._lib.ri_cache_length(self.core.handle, int(slot))
        if n < 0:
            raise native.fail()
        return n

    def longest(self, slots) -> int:
        """The length of the longest of these sequences."""
        s = np.asarray(slots, dtype=np.int32)
        n = self._lib.ri_cache_longest(self.core.handle, s.ctypes.data, len(s))
        if n < 0:
            raise native.fail()
        return n

    # ---- steps
    def reserve(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """Map pages for the tokens a step is about to write.  Either every sequence
        gets its pages or the cache is left as it was."""
        s, n = np.asarray(slots, dtype=np.int32), np.asarray(new_tokens, dtype=np.int32)
        native.check(self._lib.ri_cache_reserve(self.core.handle, s.ctypes.data, n.ctypes.data, len(s)))

    def commit(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """The step has written its tokens: advance the lengths, drop what fell out of a window."""
        s, n = np.asarray(slots, dtype=np.int32), np.asarray(new_tokens, dtype=np.int32)
        native.check(self._lib.ri_cache_commit(self.core.handle, s.ctypes.data, n.ctypes.data, len(s)))

    # ---- views for mixers
    def kv(self, entry: int) -> KVView:
        gi, ei = self._kv_of_entry[entry]
        g = self.groups[gi]
        return KVView(gi, g.k_pages[ei], g.v_pages[ei], g.page_size, g.need.window)

    def state(self, entry: int) -> torch.Tensor:
        return self._state[entry]

    def has_state(self, entry: int) -> bool:
        return entry in self._state

    def snapshot_state(self) -> dict[int, torch.Tensor]:
        """Copies of all state arenas (for a step that has to be run twice and count once)."""
        return {e: arena.clone() for e, arena in self._state.items()}

    def restore_state(self, snapshot: dict[int, torch.Tensor]) -> None:
        for e, saved in snapshot.items():
            self._state[e].copy_(saved)

    # ---- accounting
    def free_pages(self) -> list[int]:
        return [g.pool.free_count for g in self.groups]

    def check_consistent(self) -> None:
        """No slot lost or held twice; no page lost, held twice or held by a free slot."""
        native.check(self._lib.ri_cache_check(self.core.handle))


__all__ = ["Cache", "KVNeed", "StateNeed", "KVGroup", "KVView", "PAGE_SIZE", "UNMAPPED"]
