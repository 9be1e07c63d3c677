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

import itertools

import numpy as np
import torch

from .. import profiler
from ..cache import native as cache_native
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


def _one_token_wanted(e: StepEntry) -> bool:
    """One token whose logits are wanted: the entry of a decode step."""
    if len(e.tokens) != 1:
        return False
    return e.want == "last" or e.want == "all" or (not isinstance(e.want, str) and wanted_indices(1, e.want) == [0])


class _Staging:
    """A few pinned host buffers used in turn, so that a step's layout can be written
    while the copy of the one before may still be in flight."""

    def __init__(self, capacity: int, device, depth: int = 4):
        self.capacity, self.device, self.turn = capacity, device, 0
        self.host = [torch.empty(capacity, dtype=torch.int32, pin_memory=True) for _ in range(depth)]
        self.views = [h.numpy() for h in self.host]            # the same memory, for numpy to fill
        self.events = [None] * depth
        self.dev = torch.zeros(capacity, dtype=torch.int32, device=device)

    def begin(self, n: int) -> np.ndarray:
        """The next host buffer's first ``n`` words, free to be written."""
        i = self.turn
        if self.events[i] is not None:
            self.events[i].synchronize()
        return self.views[i][:n]

    def upload(self, n: int) -> torch.Tensor:
        """Send what ``begin`` handed out; returns the device buffer."""
        i = self.turn
        self.turn = (i + 1) % len(self.host)
        self.dev[:n].copy_(self.host[i][:n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.events[i] = ev
        return self.dev


class _DecodeGraph:
    """One captured decode step for a fixed number of sequences: the kernels of the whole model as
    one HIP graph, replayed with fresh tokens, positions and page tables in the same buffers."""

    def __init__(self, batch: int, device):
        self.batch = batch
        self.staging = None          # its own buffers: their addresses are part of the graph
        self.graph = None
        self.ctx = None
        self.logits = None


def _decode_bound(cache, longest: int) -> int:
    """The bound on the sequences' lengths that sizes a decode step's launches: a power of two of tokens,
    1,024 at least, the cache's limit at most."""
    return min(cache.max_seq_len, max(1024, 1 << (longest - 1).bit_length()))


# Graphs an engine keeps: one per batch size and bound that a step has had.  A batch that shrinks as its
# sequences end passes through every size below its first, and each graph holds the step's buffers (the
# logits of its batch among them); past this many the graph that has gone unused the longest is dropped and
# captured again if its size comes back.
MAX_GRAPHS = 96


class Engine:
    """A model, its cache, and the step function over them.

    With ``use_graphs`` a step in which every sequence brings one token and wants its logits runs
    as a HIP graph captured once per batch size and bound on the sequence length: the launches of
    a decode step cost more than its kernels otherwise.  Page tables then have the cache's full
    width and the attention grid is sized for the bound; the results are the same."""

    def __init__(self, model, cache, use_graphs: bool = False, capture_after: int = 0):
        self.model, self.cache = model, cache
        self.device = model.rt.device
        self.use_graphs = use_graphs
        # Decode steps of a batch size and bound run this many times with host launches before their graph is
        # captured.  Capturing costs what 3 to 5 replays take (6 ms at Qwen3-0.6B sizes, 10 to 17 at Qwen3-8B
        # sizes), and a batch whose sequences end at different times passes through every size below its first,
        # some for a step or two; a replay saves a small model half of a step with host launches (1.3 against 2.4
        # ms) and a large one a few per cent (3.35 against 3.5), so only a large model's short-lived sizes are
        # better left without a graph.  0: capture at the first step of a size.
        self.capture_after = int(capture_after)
        self._seen: dict[tuple[int, int], int] = {}
        self._staging = None
        self._graphs: dict[tuple[int, int], _DecodeGraph] = {}       # in order of last use
        self.max_graphs = MAX_GRAPHS
        self.keep_graphs = False     # keep what was captured beside what is replayed, so that its nodes can be counted

    def _stage(self, n: int) -> _Staging:
        if self._staging is None or self._staging.capacity < n:
            cap = max(1 << 16, 1 << (n - 1).bit_length())
            self._staging = _Staging(cap, self.device)
        return self._staging

    def build_context(self, entries: Sequence[StepEntry], staging: _Staging | None = None,
                      full_width: bool = False, grid_len: int | None = None) -> StepContext:
        """Reserve the step's pages and send its layout to the device: one block of int32 words
        (tokens, sequence and position of each, sequence starts, slots, lengths after the step,
        wanted rows, a page table per key/value group), laid out by the cache's native side
        straight into a pinned buffer."""
        cache = self.cache
        B = len(entries)
        if B == 0:
            raise ShapeError("a step needs at least one entry")
        slots = [e.slot for e in entries]
        counts = [len(e.tokens) for e in entries]
        for b, (e, n) in enumerate(zip(entries, counts)):
            if n < 1:
                raise ShapeError(f"entry {b} (slot {e.slot}) brings no token")
        T = sum(counts)
        starts = [cache.length(s) for s in slots]
        cu, want = [0], []
        for e, n in zip(entries, counts):
            want.extend(cu[-1] + i for i in wanted_indices(n, e.want))
            cu.append(cu[-1] + n)
        tokens = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int64, count=T)
        if T and (tokens.min() < 0 or tokens.max() >= self.model.spec.vocab_size):
            bad = int(tokens[(tokens < 0) | (tokens >= self.model.spec.vocab_size)][0])
            raise ShapeError(f"token id {bad} is outside the vocabulary of {self.model.spec.vocab_size}")
        tokens = tokens.astype(np.int32)
        cache.reserve(slots, counts)
        max_len = max(s + n for s, n in zip(starts, counts))
        width = cache.max_pages_per_slot if full_width else -(-max_len // cache.page_size)
        G = len(cache.groups)
        capacity = 3 * (T + 4) + (B + 5) + 2 * (B + 4) + (len(want) + 4) + G * (B * width + 4)
        stage = staging or self._stage(capacity)
        words = stage.begin(capacity)
        offsets = np.empty(7 + G, dtype=np.int64)
        s_arr, c_arr, w_arr = (np.asarray(a, dtype=np.int32) for a in (slots, counts, want))
        used = cache_native.lib().ri_cache_plan_step(
            cache.core.handle, s_arr.ctypes.data, c_arr.ctypes.data, B, tokens.ctypes.data, w_arr.ctypes.data, len(want),
            self.model.spec.vocab_size, width, words.ctypes.data, capacity, offsets.ctypes.data)
        if used < 0:
            raise ShapeError(cache_native.lib().ri_last_error().decode())
        dev = stage.upload(used)
        off = offsets.tolist()

        def piece(i, n):
            return dev[off[i]:off[i] + n]

        # A decode step launched from the host gets the bound a graph of it would have: kernels that choose
        # their form by the bound then choose alike either way, and a step's result does not depend on
        # whether it ran as a graph.
        if not full_width and max(counts) == 1:
            max_len = _decode_bound(cache, max_len)
        ctx = StepContext(T=T, B=B, new_counts=counts, slot_list=slots, starts=starts,
                          tokens=piece(0, T), tok_seq=piece(1, T), tok_pos=piece(2, T), cu_seqlens=piece(3, B + 1),
                          slots=piece(4, B), len_after=piece(5, B), want_rows=piece(6, len(want)),
                          n_want=len(want), max_new=max(counts),
                          max_len=grid_len or (cache.max_seq_len if full_width else max_len))
        ctx.page_tables = [piece(7 + gi, B * width).view(B, width) for gi in range(G)]
        return ctx

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run one step; float32 logits ``[n_want, vocab]`` on the device, in the order of
        the entries and of each entry's wanted places.  (With graphs the logits of a decode step
        live in the graph's own buffer and are overwritten by the next decode step of that size.)"""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        # (section timers read events around the kernels, which a captured graph does not hold)
        if self.use_graphs and not profiler.enabled() and entries and all(_one_token_wanted(e) for e in entries):
            return self._graph_step(entries)
        ctx = self.build_context(entries)
        logits = self.model.forward(ctx, self.cache)
        self.cache.commit(ctx.slot_list, ctx.new_counts)
        return logits

    def _graph_step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        batch = len(entries)
        # A graph's launches are sized for sequences up to a power of two of tokens (1,024 at least, the
        # cache's limit at most): the attention kernels launch a workgroup per chunk of keys that might be
        # there, and a cache that allows long sequences must not make short ones pay for that.  A batch
        # gets the next graph when its longest sequence grows past the bound (capturing one costs about
        # as much as two or three steps).  Finer bounds were tried and gained nothing: the workgroups of
        # the empty chunks come last in the grid and cost little there.
        slots = np.fromiter((e.slot for e in entries), dtype=np.int32, count=batch)
        bound = _decode_bound(self.cache, self.cache.longest(slots) + 1)
        dg = self._graphs.pop((batch, bound), None)
        if dg is None and self.capture_after > 0:
            if len(self._seen) > 8 * max(1, self.max_graphs):
                self._seen.clear()
            seen = self._seen[(batch, bound)] = self._seen.get((batch, bound), 0) + 1
            if seen <= self.capture_after:                   # not yet worth a graph: the step with host launches
                ctx = self.build_context(entries)
                logits = self.model.forward(ctx, self.cache)
                self.cache.commit(ctx.slot_list, ctx.new_counts)
                return logits
        if dg is not None:
            self._graphs[(batch, bound)] = dg                # the most recently used sits last
        else:
            while len(self._graphs) >= max(1, self.max_graphs):
                self._graphs.pop(next(iter(self._graphs)))   # the one unused the longest
            dg = self._graphs[(batch, bound)] = _DecodeGraph(batch, self.device)
            width = self.cache.max_pages_per_slot
            need = 7 * (batch + 5) + len(self.cache.groups) * (batch * width + 4)
            dg.staging = _Staging(need, self.device)
        if dg.graph is not None:
            return self._replay(dg, entries, slots)
        # the layout of a decode step depends on the batch size alone, so the buffers a captured
        # graph reads are refilled in place
        ctx = self.build_context(entries, staging=dg.staging, full_width=True, grid_len=bound)
        # once eagerly (libraries set themselves up outside the capture), then capture; writing
        # the same keys and values to the same places twice changes nothing, and per-sequence
        # state is put back to where it was before the rehearsal
        saved = self.cache.snapshot_state()
        self.model.forward(ctx, self.cache)
        self.cache.restore_state(saved)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph(keep_graph=True) if self.keep_graphs else torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            dg.logits = self.model.forward(ctx, self.cache)
        dg.graph, dg.ctx = graph, ctx
        dg.graph.replay()
        self.cache.commit(ctx.slot_list, ctx.new_counts)
        return dg.logits

    def _replay(self, dg: _DecodeGraph, entries: Sequence[StepEntry] | None, slots: np.ndarray,
                ids_dev: torch.Tensor | None = None) -> torch.Tensor:
        """A decode step whose graph exists: reserve the pages, write the step's layout into the buffers the
        graph reads, replay.  The same layout as ``build_context`` makes, without the objects a first run
        needs (at 64 sequences the host's share of a step is a few per cent of it).  With ``ids_dev`` the
        tokens are int32 ids already on the device (what the step before picked): they are copied into the
        layout there, after its other pieces have come from the host."""
        cache, batch = self.cache, dg.batch
        vocab = self.model.spec.vocab_size
        if ids_dev is None:
            tokens = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=batch)
            if tokens.min() < 0 or tokens.max() >= vocab:
                bad = int(tokens[(tokens < 0) | (tokens >= vocab)][0])
                raise ShapeError(f"token id {bad} is outside the vocabulary of {vocab}")
            tokens = tokens.astype(np.int32)
        else:
            if ids_dev.dtype != torch.int32 or ids_dev.shape != (batch,) or ids_dev.device != dg.ctx.tokens.device:
                raise ShapeError(f"the ids of {batch} sequences on the device: got {tuple(ids_dev.shape)} {ids_dev.dtype}")
            tokens = np.zeros(batch, dtype=np.int32)         # their place in the layout; the ids follow on the device
        ones = np.ones(batch, dtype=np.int32)
        want = np.arange(batch, dtype=np.int32)
        cache.reserve(slots, ones)
        width, groups = cache.max_pages_per_slot, len(cache.groups)
        capacity = 3 * (batch + 4) + (batch + 5) + 2 * (batch + 4) + (batch + 4) + groups * (batch * width + 4)
        words = dg.staging.begin(capacity)
        offsets = np.empty(7 + groups, dtype=np.int64)
        used = cache_native.lib().ri_cache_plan_step(
            cache.core.handle, slots.ctypes.data, ones.ctypes.data, batch, tokens.ctypes.data, want.ctypes.data, batch,
            vocab, width, words.ctypes.data, capacity, offsets.ctypes.data)
        if used < 0:
            raise ShapeError(cache_native.lib().ri_last_error().decode())
        dg.staging.upload(used)
        if ids_dev is not None:
            dg.ctx.tokens.copy_(ids_dev)                     # in stream order: after the layout, before the graph
        dg.graph.replay()
        cache.commit(slots, ones)
        return dg.logits

    def graph_launches(self) -> dict:
        """``{(batch, bound): kernel nodes}`` of the captured decode steps: the launches a step of that size
        costs.  Only for graphs captured while ``keep_graphs`` was set (measurement)."""
        import ctypes
        hip = ctypes.CDLL("libamdhip64.so")
        out = {}
        for key, dg in self._graphs.items():
            raw = getattr(dg.graph, "raw_cuda_graph", None) if dg.graph is not None else None
            try:
                handle = ctypes.c_void_p(raw()) if raw else None
            except RuntimeError:                 # captured without keep_graphs
                handle = None
            if not handle:
                continue
            n = ctypes.c_size_t(0)
            if hip.hipGraphGetNodes(handle, None, ctypes.byref(n)) != 0:
                continue
            nodes = (ctypes.c_void_p * n.value)()
            hip.hipGraphGetNodes(handle, nodes, ctypes.byref(n))
            kernels = 0
            for node in nodes:
                kind = ctypes.c_int(-1)
                if hip.hipGraphNodeGetType(ctypes.c_void_p(node), ctypes.byref(kind)) == 0 and kind.value == 0:
                    kernels += 1                 # hipGraphNodeTypeKernel
            out[key] = kernels
        return out

    def decode_on_device(self, slots: Sequence[int], ids_dev: torch.Tensor) -> torch.Tensor | None:
        """A decode step (one token per sequence, logits of every one) whose tokens are int32 ids on the device,
        so that the host need not have read them: the generation loop launches a step with what the step
        before picked and reads those picks while it runs.  Returns None where there is no captured graph for
        this step's size yet (or no graphs at all): the caller then takes ``step`` with the tokens themselves."""
        if not self.use_graphs or profiler.enabled() or len(slots) == 0:
            return None
        slots = np.asarray(slots, dtype=np.int32)
        key = (len(slots), _decode_bound(self.cache, self.cache.longest(slots) + 1))
        dg = self._graphs.get(key)
        if dg is None or dg.graph is None:
            return None
        self._graphs[key] = self._graphs.pop(key)            # the most recently used sits last
        return self._replay(dg, None, slots, ids_dev)
