// The host side of the cache and of a step's layout: which sequence holds which slot, which pages a
// slot holds in every pool, how long every sequence is, and the block of int32 words that tells the
// kernels of a step where everything lies.  No device code and no device call: this is bookkeeping that
// runs between the steps, and it runs once per step whatever the batch, so it is written where a step's
// few thousand integers cost microseconds.
//
// The reference keeps one page table per layer, hands out page 0 first, advances every sequence by the
// same count and can only reset the whole cache (src/kvcache.rs:51, :106-135, :185-196).  Here a pool
// serves all layers of one key/value geometry, sequences advance by their own counts, a slot gives its
// pages back when its sequence ends, and a pool with a window gives pages back as soon as no later query
// can see them.
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "api.h"
#include "common.h"

namespace {

constexpr int32_t UNMAPPED = -1;

struct PagePool {
    int num_pages, page_size, num_slots, max_pages_per_slot, window;   // window 0: every key stays
    std::vector<int32_t> free_list;                                    // taken from the back: page 0 first
    std::vector<int32_t> owner;                                        // page -> slot, to catch double frees
    std::vector<int32_t> tables;                                       // [num_slots][max_pages_per_slot]

    PagePool(int pages, int psize, int slots, int per_slot, int win)
        : num_pages(pages), page_size(psize), num_slots(slots), max_pages_per_slot(per_slot), window(win),
          owner(pages, UNMAPPED), tables((size_t)slots * per_slot, UNMAPPED) {
        free_list.reserve(pages);
        for (int p = pages - 1; p >= 0; --p) free_list.push_back(p);
    }
    int32_t* row(int slot) { return tables.data() + (size_t)slot * max_pages_per_slot; }
    long capacity_per_slot() const { return (long)max_pages_per_slot * page_size; }

    int pages_needed(int slot, long before, long n) {
        const long first = before / page_size, last = std::min<long>((before + n + page_size - 1) / page_size,
                                                                     max_pages_per_slot);
        int need = 0;
        const int32_t* t = row(slot);
        for (long p = first; p < last; ++p) need += t[p] == UNMAPPED;
        return need;
    }
    // Maps pages for positions before .. before + n - 1.
    int reserve(int slot, long before, long n) {
        const long end = before + n;
        RI_REQUIRE(end <= capacity_per_slot(), "slot %d would reach %ld tokens, the cache holds %ld per sequence", slot,
                   end, capacity_per_slot());                                       // src/kvcache.rs:109-114
        int32_t* t = row(slot);
        for (long p = before / page_size; p < (end + page_size - 1) / page_size; ++p) {
            if (t[p] != UNMAPPED) continue;
            RI_REQUIRE(!free_list.empty(), "cache out of pages (%d of %d tokens in all)", num_pages, page_size);
            const int32_t page = free_list.back();
            free_list.pop_back();
            owner[page] = slot;
            t[p] = page;
        }
        return 0;
    }
    int give_back(int slot, int logical) {
        int32_t* t = row(slot);
        const int32_t page = t[logical];
        if (page == UNMAPPED) return 0;
        RI_REQUIRE(owner[page] == slot, "page %d is in slot %d's table but owned by %d", page, slot, owner[page]);
        owner[page] = UNMAPPED;
        t[logical] = UNMAPPED;
        free_list.push_back(page);
        return 0;
    }
    // Gives back the pages that no query at a position >= length can see.
    int trim_behind_window(int slot, long length) {
        if (window <= 0) return 0;
        const long first_visible = std::max<long>(0, length - window + 1);   // of the next query, at `length`
        for (long p = 0; p < first_visible / page_size && p < max_pages_per_slot; ++p)
            if (give_back(slot, (int)p)) return 1;
        return 0;
    }
    int release(int slot) {
        for (int p = 0; p < max_pages_per_slot; ++p)
            if (give_back(slot, p)) return 1;
        return 0;
    }
    int held_by(int slot) {
        int n = 0;
        const int32_t* t = row(slot);
        for (int p = 0; p < max_pages_per_slot; ++p) n += t[p] != UNMAPPED;
        return n;
    }
    // Every page is either free or in exactly one table.
    int check() {
        std::vector<int32_t> seen(num_pages, UNMAPPED);
        long held = 0;
        for (int s = 0; s < num_slots; ++s) {
            const int32_t* t = row(s);
            for (int p = 0; p < max_pages_per_slot; ++p) {
                const int32_t page = t[p];
                if (page == UNMAPPED) continue;
                RI_REQUIRE(page >= 0 && page < num_pages, "slot %d's table names page %d of %d", s, page, num_pages);
                RI_REQUIRE(seen[page] == UNMAPPED, "page %d is held twice (slots %d and %d)", page, seen[page], s);
                RI_REQUIRE(owner[page] == s, "page %d: owner %d but in slot %d's table", page, owner[page], s);
                seen[page] = s;
                ++held;
            }
        }
        std::vector<uint8_t> is_free(num_pages, 0);
        for (int32_t page : free_list) {
            RI_REQUIRE(page >= 0 && page < num_pages, "the free list names page %d of %d", page, num_pages);
            RI_REQUIRE(!is_free[page], "page %d is on the free list twice", page);
            RI_REQUIRE(seen[page] == UNMAPPED, "page %d is both free and held", page);
            is_free[page] = 1;
        }
        RI_REQUIRE((long)free_list.size() + held == num_pages, "%ld pages are lost",
                   num_pages - (long)free_list.size() - held);
        return 0;
    }
};

struct CacheCore {
    int num_slots, max_seq_len;
    std::vector<PagePool*> pools;                 // not owned: the pools outlive their cache
    std::vector<int32_t> free_slots;              // taken from the back: slot 0 first
    std::vector<uint8_t> held;
    std::vector<int64_t> lengths;

    int check_held(int slot) const {
        RI_REQUIRE(slot >= 0 && slot < num_slots, "slot %d does not exist (the cache has %d)", slot, num_slots);
        RI_REQUIRE(held[slot], "slot %d is not held (never acquired, or released already)", slot);
        return 0;
    }
};

}  // namespace

// ---------------------------------------------------------------- a pool by itself
extern "C" void* ri_pool_new(int num_pages, int page_size, int num_slots, int max_pages_per_slot, int window) {
    if (num_pages < 1 || page_size < 1 || num_slots < 1 || max_pages_per_slot < 1 || window < 0) {
        ri_set_error("page pool sizes must be positive");
        return nullptr;
    }
    return new PagePool(num_pages, page_size, num_slots, max_pages_per_slot, window);
}
extern "C" void ri_pool_delete(void* pool) { delete (PagePool*)pool; }
extern "C" int32_t* ri_pool_tables(void* pool) { return ((PagePool*)pool)->tables.data(); }
extern "C" int ri_pool_free_count(void* pool) { return (int)((PagePool*)pool)->free_list.size(); }
extern "C" int ri_pool_pages_needed(void* pool, int slot, long before, long n) {
    return ((PagePool*)pool)->pages_needed(slot, before, n);
}
extern "C" int ri_pool_reserve(void* pool, int slot, long before, long n) { return ((PagePool*)pool)->reserve(slot, before, n); }
extern "C" int ri_pool_trim(void* pool, int slot, long length) { return ((PagePool*)pool)->trim_behind_window(slot, length); }
extern "C" int ri_pool_release(void* pool, int slot) { return ((PagePool*)pool)->release(slot); }
extern "C" int ri_pool_check(void* pool) { return ((PagePool*)pool)->check(); }

// ---------------------------------------------------------------- slots, lengths and the pools together
extern "C" void* ri_cache_new(void* const* pools, int num_pools, int num_slots, int max_seq_len) {
    if (num_slots < 1 || max_seq_len < 1 || num_pools < 0) {
        ri_set_error("a cache needs at least one slot and a positive sequence length");
        return nullptr;
    }
    CacheCore* c = new CacheCore;
    c->num_slots = num_slots;
    c->max_seq_len = max_seq_len;
    for (int i = 0; i < num_pools; ++i) c->pools.push_back((PagePool*)pools[i]);
    for (int s = num_slots - 1; s >= 0; --s) c->free_slots.push_back(s);
    c->held.assign(num_slots, 0);
    c->lengths.assign(num_slots, 0);
    return c;
}
extern "C" void ri_cache_delete(void* cache) { delete (CacheCore*)cache; }

extern "C" int ri_cache_acquire(void* cache) {
    CacheCore* c = (CacheCore*)cache;
    if (c->free_slots.empty()) {
        ri_set_error("no free slot: all %d are held by live sequences", c->num_slots);
        return -1;
    }
    const int slot = c->free_slots.back();
    c->free_slots.pop_back();
    c->held[slot] = 1;
    c->lengths[slot] = 0;
    return slot;
}

extern "C" int ri_cache_release(void* cache, int slot) {
    CacheCore* c = (CacheCore*)cache;
    if (c->check_held(slot)) return 1;
    c->held[slot] = 0;
    c->free_slots.push_back(slot);
    c->lengths[slot] = 0;
    for (PagePool* p : c->pools)
        if (p->release(slot)) return 1;
    return 0;
}

extern "C" int ri_cache_is_held(void* cache, int slot) {
    CacheCore* c = (CacheCore*)cache;
    return slot >= 0 && slot < c->num_slots && c->held[slot];
}
extern "C" int ri_cache_check_held(void* cache, int slot) { return ((CacheCore*)cache)->check_held(slot); }
extern "C" int ri_cache_free_slots(void* cache) { return (int)((CacheCore*)cache)->free_slots.size(); }

extern "C" long ri_cache_length(void* cache, int slot) {
    CacheCore* c = (CacheCore*)cache;
    if (c->check_held(slot)) return -1;
    return (long)c->lengths[slot];
}

// The longest of these sequences, or -1 (one call for a whole batch instead of one per sequence).
extern "C" long ri_cache_longest(void* cache, const int32_t* slots, int n) {
    CacheCore* c = (CacheCore*)cache;
    long longest = 0;
    for (int i = 0; i < n; ++i) {
        if (c->check_held(slots[i])) return -1;
        longest = std::max(longest, (long)c->lengths[slots[i]]);
    }
    return longest;
}

// Maps pages for the tokens a step is about to write: either every sequence gets its pages in every
// pool, or the cache is left as it was.
extern "C" int ri_cache_reserve(void* cache, const int32_t* slots, const int32_t* counts, int n) {
    CacheCore* c = (CacheCore*)cache;
    std::vector<uint8_t> in_step(c->num_slots, 0);
    for (int i = 0; i < n; ++i) {
        if (c->check_held(slots[i])) return 1;
        RI_REQUIRE(!in_step[slots[i]], "a slot appears twice in one step");
        in_step[slots[i]] = 1;
        RI_REQUIRE(counts[i] >= 1, "slot %d: a step needs at least one token", slots[i]);
        RI_REQUIRE(c->lengths[slots[i]] + counts[i] <= c->max_seq_len,
                   "slot %d would reach %ld tokens, the cache holds %d per sequence", slots[i],
                   (long)(c->lengths[slots[i]] + counts[i]), c->max_seq_len);
    }
    for (PagePool* p : c->pools) {
        long want = 0;
        for (int i = 0; i < n; ++i) want += p->pages_needed(slots[i], c->lengths[slots[i]], counts[i]);
        RI_REQUIRE(want <= (long)p->free_list.size(),
                   "cache out of pages: the step needs %ld more, %ld of %d are free (%d tokens each)", want,
                   (long)p->free_list.size(), p->num_pages, p->page_size);
    }
    for (PagePool* p : c->pools)
        for (int i = 0; i < n; ++i)
            if (p->reserve(slots[i], c->lengths[slots[i]], counts[i])) return 1;
    return 0;
}

// The step has written its tokens: the lengths advance, and what fell out of a window goes back.
extern "C" int ri_cache_commit(void* cache, const int32_t* slots, const int32_t* counts, int n) {
    CacheCore* c = (CacheCore*)cache;
    for (int i = 0; i < n; ++i) {
        if (c->check_held(slots[i])) return 1;
        c->lengths[slots[i]] += counts[i];
        for (PagePool* p : c->pools)
            if (p->trim_behind_window(slots[i], c->lengths[slots[i]])) return 1;
    }
    return 0;
}

// No slot lost or held twice, no page lost, held twice or held by a free slot.
extern "C" int ri_cache_check(void* cache) {
    CacheCore* c = (CacheCore*)cache;
    std::vector<uint8_t> is_free(c->num_slots, 0);
    for (int32_t s : c->free_slots) {
        RI_REQUIRE(s >= 0 && s < c->num_slots && !is_free[s], "slot %d is on the free list twice", s);
        RI_REQUIRE(!c->held[s], "slot %d is both free and held", s);
        is_free[s] = 1;
    }
    long held = 0;
    for (int s = 0; s < c->num_slots; ++s) held += c->held[s];
    RI_REQUIRE(held + (long)c->free_slots.size() == c->num_slots, "a slot is lost");
    for (PagePool* p : c->pools) {
        if (p->check()) return 1;
        for (int s = 0; s < c->num_slots; ++s)
            RI_REQUIRE(c->held[s] || p->held_by(s) == 0, "slot %d is free but still holds pages", s);
    }
    return 0;
}

// ---------------------------------------------------------------- the layout of a step
// Everything the kernels read of a step's layout, as one block of int32 words with every piece on a
// 16-byte boundary, in this order: the tokens, each token's sequence (its index in this step) and
// position, where each sequence starts among the tokens (n + 1 words), the slots, the lengths after the
// step, the wanted rows, then one page table [n][width] per pool.  Positions are the cache lengths.
// offsets: 7 + pools words, each piece's place in the block.  Returns the words used, -1 on error.
// Call after ri_cache_reserve (the tables then hold the step's pages) and before ri_cache_commit.
extern "C" long ri_cache_plan_step(void* cache, const int32_t* slots, const int32_t* counts, int n,
                                   const int32_t* tokens, const int32_t* want_rows, int n_want, int vocab, int width,
                                   int32_t* words, long capacity, int64_t* offsets) {
    CacheCore* c = (CacheCore*)cache;
    long total = 0;
    for (int i = 0; i < n; ++i) {
        if (c->check_held(slots[i])) return -1;
        if (counts[i] < 1) {
            ri_set_error("entry %d (slot %d) brings no token", i, slots[i]);
            return -1;
        }
        total += counts[i];
    }
    for (long t = 0; t < total; ++t)
        if (tokens[t] < 0 || tokens[t] >= vocab) {                                   // src/ops/embedding.rs:20-22
            ri_set_error("token id %d is outside the vocabulary of %d", tokens[t], vocab);
            return -1;
        }
    for (int w = 0; w < n_want; ++w)
        if (want_rows[w] < 0 || want_rows[w] >= total) {
            ri_set_error("wanted row %d is outside the step's %ld tokens", want_rows[w], total);
            return -1;
        }
    const int pools = (int)c->pools.size();
    const long sizes[7] = {total, total, total, (long)n + 1, n, n, n_want};
    long at = 0;
    for (int p = 0; p < 7 + pools; ++p) {
        offsets[p] = at;
        const long size = p < 7 ? sizes[p] : (long)n * width;
        at += (size + 3) / 4 * 4;
    }
    if (at > capacity) {
        ri_set_error("the step's layout takes %ld words, the buffer has %ld", at, capacity);
        return -1;
    }
    int32_t* tok = words + offsets[0];
    int32_t* seq = words + offsets[1];
    int32_t* pos = words + offsets[2];
    int32_t* cu = words + offsets[3];
    int32_t* slot_out = words + offsets[4];
    int32_t* len_after = words + offsets[5];
    memcpy(tok, tokens, (size_t)total * sizeof(int32_t));
    long t = 0;
    cu[0] = 0;
    for (int i = 0; i < n; ++i) {
        const int64_t start = c->lengths[slots[i]];
        for (int j = 0; j < counts[i]; ++j, ++t) {
            seq[t] = i;
            pos[t] = (int32_t)(start + j);
        }
        cu[i + 1] = (int32_t)t;
        slot_out[i] = slots[i];
        len_after[i] = (int32_t)(start + counts[i]);
    }
    if (n_want) memcpy(words + offsets[6], want_rows, (size_t)n_want * sizeof(int32_t));
    for (int p = 0; p < pools; ++p) {
        PagePool* pool = c->pools[p];
        if (width > pool->max_pages_per_slot) {
            ri_set_error("a page table of %d columns from a pool with %d pages a slot", width, pool->max_pages_per_slot);
            return -1;
        }
        int32_t* table = words + offsets[7 + p];
        for (int i = 0; i < n; ++i) memcpy(table + (size_t)i * width, pool->row(slots[i]), (size_t)width * sizeof(int32_t));
    }
    return at;
}
