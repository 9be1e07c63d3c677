"""The cache's accounting (no GPU): no slot or page lost, held twice or freed twice."""
import random

import pytest
import torch

from rust_inference_amd.cache import Cache, KVNeed, PagePool, SlotAllocator, StateNeed
from rust_inference_amd.errors import CacheError


def make(needs=None, slots=4, max_tokens=256, max_seq_len=128):
    needs = needs or [KVNeed(2, 16), KVNeed(2, 16)]
    return Cache(needs, slots, max_tokens, max_seq_len, dtype=torch.float32, device="cpu")


def test_slots_are_reused_and_never_held_or_freed_twice():
    a = SlotAllocator(2)
    s0, s1 = a.acquire(), a.acquire()
    assert (s0, s1) == (0, 1)
    with pytest.raises(CacheError, match="no free slot"):
        a.acquire()
    a.release(s0)
    with pytest.raises(CacheError, match="not held"):
        a.release(s0)
    with pytest.raises(CacheError, match="does not exist"):
        a.release(7)
    assert a.acquire() == s0 and a.free_count == 0


def test_pages_are_mapped_lazily_vector_of_the_reference():
    # src/kvcache.rs:216-227: 4 pages, 1 sequence, 3 pages per sequence
    p = PagePool(num_pages=4, page_size=32, num_slots=1, max_pages_per_slot=3)
    p.reserve(0, 0, 1)
    assert p.tables[0].tolist() == [0, -1, -1]
    p.reserve(0, 0, 33)
    assert p.tables[0].tolist() == [0, 1, -1] and p.free_count == 2
    with pytest.raises(CacheError, match="per sequence"):
        p.reserve(0, 0, 97)
    p.release(0)
    assert p.free_count == 4
    p.check_consistent()


def test_lengths_are_per_slot_and_release_gives_pages_back():
    c = make()
    a, b = c.acquire(), c.acquire()
    c.reserve([a, b], [33, 2])
    c.commit([a, b], [33, 2])
    assert (c.length(a), c.length(b)) == (33, 2) and c.free_pages() == [8 - 3]
    c.reserve([a], [1])
    c.commit([a], [1])
    assert c.length(a) == 34 and c.free_pages() == [5]         # position 33 lies in a page already mapped
    c.release(b)
    assert c.free_pages() == [6]
    with pytest.raises(CacheError, match="not held"):
        c.length(b)
    with pytest.raises(CacheError, match="not held"):
        c.release(b)
    b2 = c.acquire()
    assert b2 == b and c.length(b2) == 0                       # the slot comes back empty
    c.check_consistent()


def test_a_step_that_does_not_fit_changes_nothing():
    c = make(slots=3, max_tokens=96, max_seq_len=96)           # 3 pages
    a, b = c.acquire(), c.acquire()
    with pytest.raises(CacheError, match="out of pages"):
        c.reserve([a, b], [40, 40])                            # 2 + 2 pages
    assert c.free_pages() == [3] and c.length(a) == 0
    with pytest.raises(CacheError, match="per sequence"):
        c.reserve([a], [97])
    with pytest.raises(CacheError, match="twice"):
        c.reserve([a, a], [1, 1])
    with pytest.raises(CacheError, match="at least one token"):
        c.reserve([a], [0])
    c.check_consistent()


def test_groups_with_different_needs_have_storage_of_their_own():
    c = make(needs=[KVNeed(2, 16), KVNeed(2, 16, window=40), KVNeed(1, 32), KVNeed(2, 16), StateNeed((5,)), None])
    assert len(c.groups) == 3
    assert [g.entries for g in c.groups] == [[0, 3], [1], [2]]
    assert c.kv(3).k_pages.shape == (8, 2, 32, 16) and c.kv(2).k_pages.shape == (8, 1, 32, 32)
    assert c.kv(3).v_pages.shape == (8, 2, 16, 32)
    assert c.kv(0).k_pages.data_ptr() != c.kv(3).k_pages.data_ptr()
    assert c.state(4).shape == (4, 5) and c.has_state(4) and not c.has_state(0)
    s = c.acquire()
    c.reserve([s], [100])
    c.commit([s], [100])
    # all keys: 4 pages held; window of 40 at length 100: the next query (position 100) sees 61..100,
    # so the page of positions 0..31 went back
    assert c.free_pages() == [4, 5, 4]
    assert c.groups[1].pool.tables[s][:4].tolist() == [-1, 1, 2, 3]
    c.release(s)
    assert c.free_pages() == [8, 8, 8]
    c.check_consistent()


def test_state_rows_are_zero_for_a_new_sequence():
    c = make(needs=[StateNeed((3,))])
    s = c.acquire()
    c.state(0)[s] += 5.0
    c.release(s)
    assert c.acquire() == s and torch.equal(c.state(0)[s], torch.zeros(3))


def test_random_traffic_loses_nothing():
    rng = random.Random(0)
    c = make(needs=[KVNeed(1, 16), KVNeed(1, 16, window=48)], slots=6, max_tokens=32 * 20, max_seq_len=200)
    live = {}
    for _ in range(600):
        op = rng.random()
        if op < 0.3 and len(live) < 6:
            live[c.acquire()] = 0
        elif op < 0.5 and live:
            s = rng.choice(list(live))
            c.release(s)
            del live[s]
        elif live:
            group = rng.sample(list(live), rng.randint(1, len(live)))
            counts = [rng.randint(1, 40) for _ in group]
            try:
                c.reserve(group, counts)
            except CacheError:
                continue
            c.commit(group, counts)
            for s, n in zip(group, counts):
                live[s] += n
        c.check_consistent()
        assert all(c.length(s) == n for s, n in live.items())
    for s in list(live):
        c.release(s)
    c.check_consistent()
    assert c.free_pages() == [20, 20] and c.slots.free_count == 6
