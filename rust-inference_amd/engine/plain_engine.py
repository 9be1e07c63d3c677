"""The whole model on the CPU: the step function over the plain forms of the parts.

The reference's CPU path is a float32-compute model: activations are float32, weights are decoded from what
they are stored in and summed in float32, the cache is float32 (src/ops/mod.rs:36-41; src/cpu/linear.rs:119-130,
:158-198; src/models/qwen3.rs:201-202).  This engine is that path for the parts that have a plain form (the
library's own do: each runs on the scalar C++ twins of the kernels, csrc/plain).  It is chosen by name
(``Model.load(..., device="cpu")``, ``runner --device cpu``), never fallen back to; it exists to read a
checkpoint's output without a GPU and as a second opinion beside the kernels, not for speed.

The cache's bookkeeping is the GPU engine's (slots, pages, reservation, the writer of a step's layout: native
host code); only the storage differs: float32 numpy arrays.  ``step`` has the interface of ``Engine.step`` and
returns float32 logits on the CPU, which the generation loop samples with the host sampler.
"""
from __future__ import annotations

import itertools
from typing import Sequence

import numpy as np
import torch

from ..cache import Cache, KVNeed
from ..cache import native as cache_native
from ..errors import ConfigError, ShapeError
from ..parts.context import StepContext
from .step import StepEntry, wanted_indices


class PlainEngine:
    def __init__(self, model, num_slots: int, max_tokens: int, max_seq_len: int):
        self.model = model
        needs = model.cache_needs()
        for e, need in enumerate(needs):
            if need is not None and not isinstance(need, KVNeed):
                raise ConfigError(f"cache entry {e} keeps {need!r}: the plain backend keeps keys and values only")
        self.cache = Cache(needs, num_slots, max_tokens, max_seq_len, dtype=torch.float32, device="cpu", allocate=False)
        self.stores = {}
        for gi, g in enumerate(self.cache.groups):
            n = g.need
            for e in g.entries:
                k = np.zeros((g.pool.num_pages, n.kv_heads, g.page_size, n.head_dim), dtype=np.float32)
                v = np.zeros((g.pool.num_pages, n.kv_heads, n.head_dim, g.page_size), dtype=np.float32)
                self.stores[e] = ((k, v), gi)

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        cache, vocab = self.cache, self.model.spec.vocab_size
        B = len(entries)
        if B == 0:
            raise ShapeError("a step needs at least one entry")
        slots = [e.slot for e in entries]
        counts = [len(e.tokens) for e in entries]
        if min(counts) < 1:
            raise ShapeError("an entry brings no token")
        T = sum(counts)
        starts = [cache.length(s) for s in slots]
        cu, want = [0], []
        for e, n in zip(entries, counts):
            want.extend(cu[-1] + i for i in wanted_indices(n, e.want))
            cu.append(cu[-1] + n)
        tokens = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int64, count=T)
        if tokens.min() < 0 or tokens.max() >= vocab:
            bad = int(tokens[(tokens < 0) | (tokens >= vocab)][0])
            raise ShapeError(f"token id {bad} is outside the vocabulary of {vocab}")
        tokens = tokens.astype(np.int32)
        cache.reserve(slots, counts)
        width = -(-max(s + n for s, n in zip(starts, counts)) // cache.page_size)
        G = len(cache.groups)
        capacity = 3 * (T + 4) + (B + 5) + 2 * (B + 4) + (len(want) + 4) + G * (B * width + 4)
        words = np.zeros(capacity, dtype=np.int32)
        offsets = np.empty(7 + G, dtype=np.int64)
        s_arr, c_arr, w_arr = (np.asarray(a, dtype=np.int32) for a in (slots, counts, want))
        used = cache_native.lib().ri_cache_plan_step(
            cache.core.handle, s_arr.ctypes.data, c_arr.ctypes.data, B, tokens.ctypes.data, w_arr.ctypes.data, len(want),
            vocab, width, words.ctypes.data, capacity, offsets.ctypes.data)
        if used < 0:
            raise ShapeError(cache_native.lib().ri_last_error().decode())
        off = offsets.tolist()

        def piece(i, n):
            return words[off[i]:off[i] + n]

        ctx = StepContext(T=T, B=B, new_counts=counts, slot_list=slots, starts=starts, tokens=piece(0, T),
                          tok_seq=piece(1, T), tok_pos=piece(2, T), cu_seqlens=piece(3, B + 1), slots=piece(4, B),
                          len_after=piece(5, B), want_rows=piece(6, len(want)), n_want=len(want), max_new=max(counts),
                          max_len=max(s + n for s, n in zip(starts, counts)))
        tables = [piece(7 + gi, B * width).reshape(B, width) for gi in range(G)]
        logits = self.model.plain_forward(ctx, self.stores, tables).reshape(len(want), vocab)
        cache.commit(slots, counts)
        return torch.from_numpy(np.ascontiguousarray(logits, dtype=np.float32))
