"""The step function: one batch of sequences, the tokens each brings, logits at the wanted places.

A step runs only the tokens it is given, all sequences as one flattened batch, from
what earlier steps left in the cache.  Prompts go through in one step (unequal
lengths side by side, no padding tokens exist), then one token per sequence per
step; any other cut (a prompt in pieces, several tokens in a later step) is the
same code.  Positions are the cache lengths.  The reference's forward takes a
rectangular ``[B, S]`` batch and advances every sequence by the same count
(src/models/mod.rs:36-44, src/kvcache.rs:185-187).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence, Union

import torch

from ..errors import ShapeError
from ..parts.context import StepContext

Want = Union[str, Sequence[int]]


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Want = "last"          # "last", "all", "none" or indices into ``tokens``


def wanted_indices(n: int, want: Want) -> list[int]:
    if isinstance(want, str):
        if want == "last":
            return [n - 1]
        if want == "all":
            return list(range(n))
        if want == "none":
            return []
        raise ShapeError(f"want={want!r}: expected 'last', 'all', 'none' or a list of indices")
    out = [int(i) for i in want]
    for i in out:
        if not 0 <= i < n:
            raise ShapeError(f"wanted index {i} is outside the entry's {n} tokens")
    return out


def plan_step(entries: Sequence[StepEntry], lengths: Sequence[int], vocab_size: int):
    """The host-side layout of a step: flat tokens, each token's sequence and position,
    the wanted rows.  ``lengths[i]`` is entry i's cache length before the step."""
    if not entries:
        raise ShapeError("a step needs at least one entry")
    tokens, tok_seq, tok_pos, cu, want_rows = [], [], [], [0], []
    for b, (e, start) in enumerate(zip(entries, lengths)):
        n = len(e.tokens)
        if n < 1:
            raise ShapeError(f"entry {b} (slot {e.slot}) brings no token")
        for t in e.tokens:
            if not 0 <= int(t) < vocab_size:
                raise ShapeError(f"token id {t} is outside the vocabulary of {vocab_size}")   # src/ops/embedding.rs:20-22
        base = cu[-1]
        tokens.extend(int(t) for t in e.tokens)
        tok_seq.extend([b] * n)
        tok_pos.extend(range(start, start + n))
        want_rows.extend(base + i for i in wanted_indices(n, e.want))
        cu.append(base + n)
    return tokens, tok_seq, tok_pos, cu, want_rows


class _Staging:
    """A few pinned host buffers used in turn, so that a step's layout can be written
    while the copy of the one before may still be in flight."""

    def __init__(self, capacity: int, device, depth: int = 4):
        self.capacity, self.device, self.turn = capacity, device, 0
        self.host = [torch.empty(capacity, dtype=torch.int32, pin_memory=True) for _ in range(depth)]
        self.events = [None] * depth
        self.dev = torch.zeros(capacity, dtype=torch.int32, device=device)

    def upload(self, values: list[int]) -> torch.Tensor:
        n = len(values)
        i = self.turn
        self.turn = (i + 1) % len(self.host)
        if self.events[i] is not None:
            self.events[i].synchronize()
        self.host[i][:n] = torch.tensor(values, dtype=torch.int32)
        self.dev[:n].copy_(self.host[i][:n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.events[i] = ev
        return self.dev


class Engine:
    """A model, its cache, and the step function over them."""

    def __init__(self, model, cache):
        self.model, self.cache = model, cache
        self.device = model.rt.device
        self._staging = None

    def _stage(self, n: int) -> _Staging:
        if self._staging is None or self._staging.capacity < n:
            cap = max(1 << 16, 1 << (n - 1).bit_length())
            self._staging = _Staging(cap, self.device)
        return self._staging

    def build_context(self, entries: Sequence[StepEntry], table_width: int | None = None) -> StepContext:
        cache = self.cache
        slots = [e.slot for e in entries]
        starts = [cache.length(s) for s in slots]
        counts = [len(e.tokens) for e in entries]
        tokens, tok_seq, tok_pos, cu, want_rows = plan_step(entries, starts, self.model.spec.vocab_size)
        cache.reserve(slots, counts)
        len_after = [s + n for s, n in zip(starts, counts)]
        max_len = max(len_after)
        width = table_width or -(-max_len // cache.page_size)
        pieces = [tokens, tok_seq, tok_pos, cu, slots, len_after, want_rows]
        for g in cache.groups:
            rows = g.table_rows(slots, width)
            pieces.append([p for row in rows for p in (row + [-1] * (width - len(row)))])
        flat, offsets = [], []
        for p in pieces:
            offsets.append(len(flat))
            flat.extend(p)
            flat.extend([0] * (-len(flat) % 4))           # keep every piece 16-byte aligned
        dev = self._stage(len(flat)).upload(flat)

        def piece(i, n):
            return dev[offsets[i]:offsets[i] + n]

        T, B = len(tokens), len(entries)
        ctx = StepContext(T=T, B=B, new_counts=counts, slot_list=slots, starts=starts,
                          tokens=piece(0, T), tok_seq=piece(1, T), tok_pos=piece(2, T), cu_seqlens=piece(3, B + 1),
                          slots=piece(4, B), len_after=piece(5, B), want_rows=piece(6, len(want_rows)),
                          n_want=len(want_rows), max_new=max(counts), max_len=max_len)
        ctx.page_tables = [piece(7 + gi, B * width).view(B, width) for gi in range(len(cache.groups))]
        return ctx

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run one step; float32 logits ``[n_want, vocab]`` on the device, in the order of
        the entries and of each entry's wanted places."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        ctx = self.build_context(entries)
        logits = self.model.forward(ctx, self.cache)
        self.cache.commit(ctx.slot_list, ctx.new_counts)
        return logits
