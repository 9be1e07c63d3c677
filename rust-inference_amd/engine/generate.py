"""The generation loop above the step function.

Requests (prompts as token ids) are served in batches: the sequences of a batch
start together with their prompts in one step, then take one token each per step;
a sequence that ends leaves the batch and gives its slot and pages back at once,
and the steps after it no longer carry it.  When a batch has ended the next one
starts, on the same cache, until every request is served.

Per sequence the loop is the reference's (src/bin/runner.rs:287-313): the first
token comes from the prompt's logits and counts toward ``max_new_tokens``; a stop
token is tested before it is put out, is not part of the output and is never fed
back; the last token allowed is put out but not fed.

Where the engine can take a step's tokens from the device (``decode_on_device``: captured graphs; a repetition
penalty's history is then marked on the device from those ids too), the loop runs one step ahead of what it has read: it
launches step n + 1 with the ids step n picked, still on the device, and reads step n's ids while step n + 1
runs, so that the host's share of a step (the rules below, the step's layout, the launch) hides behind the
GPU's.  A sequence whose token then turns out to be a stop token has been carried through one step too many:
that step's result for it is dropped, its slot goes back as it would have, and nobody's tokens change.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Sequence

from .. import profiler
from ..errors import CacheError, ShapeError
import torch

from ..sampling import DeviceHistory, SamplingParams, SequenceSampler, pick_batch, sample_batch
from ..sampling.batch import upload
from .step import StepEntry


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_tokens: int = 0           # tokens produced by decode steps (the reference's `generated - 1`)
    decode_seconds: float = 0.0
    decode_steps: int = 0
    batches: int = 0

    @property
    def prefill_tokens_per_second(self) -> float:
        return self.prompt_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def decode_tokens_per_second(self) -> float:
        return self.decode_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0


@dataclass
class GenerationResult:
    tokens: list                     # per request, the generated token ids (stop token not included)
    finish_reasons: list             # per request: "stop" or "length"
    stats: GenerationStats = field(default_factory=GenerationStats)


def pages_for(prompt_len: int, max_new_tokens: int, page_size: int) -> int:
    """Pages a sequence can come to hold: the last generated token is never fed, so the
    cache sees ``prompt_len + max_new_tokens - 1`` tokens at most."""
    held = prompt_len + max(max_new_tokens, 1) - 1
    return -(-held // page_size)


def plan_batches(prompt_lens: Sequence[int], max_new_tokens: int, page_size: int, total_pages: int,
                 num_slots: int, max_seq_len: int, max_batch: int | None = None) -> list[range]:
    """Cut the requests, in order, into batches that fit the cache: at most
    ``num_slots`` (and ``max_batch``) sequences whose pages fit together."""
    limit = min(num_slots, max_batch) if max_batch else num_slots
    batches, start, used = [], 0, 0
    for i, n in enumerate(prompt_lens):
        if n < 1:
            raise ShapeError(f"request {i} has an empty prompt")                       # src/bin/runner.rs:235-237
        if n + max(max_new_tokens, 1) - 1 > max_seq_len:
            raise CacheError(f"request {i}: {n} prompt tokens and {max_new_tokens} new ones exceed the "
                             f"{max_seq_len} tokens a sequence may hold")
        need = pages_for(n, max_new_tokens, page_size)
        if need > total_pages:
            raise CacheError(f"request {i} needs {need} pages, the cache has {total_pages}")
        if i > start and (i - start >= limit or used + need > total_pages):
            batches.append(range(start, i))
            start, used = i, 0
        used += need
    if start < len(prompt_lens):
        batches.append(range(start, len(prompt_lens)))
    return batches


class _Live:
    """One sequence of the running batch."""

    def __init__(self, request: int, slot: int, prompt, sampler: SequenceSampler):
        self.request, self.slot, self.prompt, self.sampler = request, slot, prompt, sampler
        self.out: list[int] = []
        self.generated = 0
        self.next_token = None
        self.reason = None


class _Flight:
    """A step that has been launched and sampled but whose picks the host has not read: its sequences, the
    ids on the device, and their copy on its way into a pinned buffer."""

    def __init__(self, members, ids, pinned, turn):
        self.members, self.ids, self.event, self.host = members, ids, None, None
        if ids.is_cuda:
            if pinned[turn] is None or pinned[turn].numel() < ids.numel():
                pinned[turn] = torch.empty(max(ids.numel(), 64), dtype=torch.int32, pin_memory=True)
            self.host = pinned[turn][:ids.numel()]
            self.host.copy_(ids, non_blocking=True)
            self.event = torch.cuda.Event()
            self.event.record()

    def read(self) -> list:
        if self.event is None:
            return self.ids.tolist()
        self.event.synchronize()
        return self.host.tolist()


def run_batch(engine, requests: Sequence[int], prompts, max_new_tokens: int, sampling,
              stop: frozenset, ignore_eos: bool, stats: GenerationStats, on_token=None) -> dict:
    """Serve one batch to the end; returns request -> (tokens, reason).  ``sampling`` is one ``SamplingParams``
    for every request, or one per request (indexed like ``prompts``)."""
    cache = engine.cache
    live = []
    of = (lambda r: sampling) if isinstance(sampling, SamplingParams) else (lambda r: sampling[r])
    penalised = any(of(r).repetition_penalty != 1.0 for r in requests)
    try:
        for r in requests:
            live.append(_Live(r, cache.acquire(), list(prompts[r]), SequenceSampler(of(r), r, prompts[r])))
    except Exception:
        for s in live:
            cache.release(s.slot)
        raise
    done = {}
    held = {s.slot for s in live}
    try:
        t0 = time.perf_counter()
        logits = engine.step([StepEntry(s.slot, s.prompt, "last") for s in live])
        history = None
        if penalised and logits.is_cuda:
            history = DeviceHistory([s.sampler for s in live], logits.shape[1], logits.device)
        with profiler.section(profiler.SAMPLING):
            picks = sample_batch(logits, [s.sampler for s in live], history)
        stats.prompt_tokens += sum(len(s.prompt) for s in live)
        stats.prefill_seconds += time.perf_counter() - t0      # includes the first sample, as in the reference
        for s, tok in zip(live, picks):
            s.next_token, s.generated = int(tok), 1
        t0 = time.perf_counter()

        def settle(s) -> bool:
            """The rules for a token that has just become known; whether the sequence goes on."""
            if not ignore_eos and s.next_token in stop:
                s.reason = "stop"                               # tested before output; not part of it
            else:
                s.out.append(s.next_token)
                if on_token is not None:
                    on_token(s.request, s.next_token)
                if s.generated >= max_new_tokens:
                    s.reason = "length"                         # put out but never fed
            if s.reason is None:
                return True
            done[s.request] = (s.out, s.reason)
            cache.release(s.slot)                               # slot and pages go back at once
            held.discard(s.slot)
            return False

        # (with a repetition penalty the loop runs ahead only where the history is kept on the device, which is then
        # marked from the ids in flight; the host sampler reads a history that the host must have written first)
        ahead = (not penalised or history is not None) and hasattr(engine, "decode_on_device")
        pinned = [None, None]
        flight = None                                           # the step whose picks the host has not read yet
        while True:
            if flight is None:
                # every sequence of `live` has a token that is known and not yet settled
                live = [s for s in live if settle(s)]
                if not live:
                    break
                logits = engine.step([StepEntry(s.slot, [s.next_token], "last") for s in live])
                for s in live:
                    s.sampler.history.append(s.next_token)
                if history is not None:
                    history.mark([s.sampler.seen_row for s in live], [s.next_token for s in live])
                with profiler.section(profiler.SAMPLING):
                    picks = pick_batch(logits, [s.sampler for s in live], history)
                for s in live:
                    s.generated += 1
                stats.decode_tokens += len(live)
                stats.decode_steps += 1
                if ahead:
                    flight = _Flight(live, picks, pinned, stats.decode_steps & 1)
                else:
                    for s, tok in zip(live, picks.tolist()):
                        s.next_token = int(tok)
                continue
            # A step is in flight.  Whoever took part in it and may have another token goes into the next step
            # with the id it picked, before the host knows that id; then the host reads the picks in flight.
            members = flight.members
            going = [i for i, s in enumerate(members) if s.reason is None and s.generated < max_new_tokens]
            logits = None
            if going:
                ids = flight.ids if len(going) == len(members) else flight.ids[upload(going, torch.int64, flight.ids.device)]
                logits = engine.decode_on_device([members[i].slot for i in going], ids)
            for s, tok in zip(members, flight.read()):
                if s.reason is None:
                    s.next_token = int(tok)
            if logits is None:                                  # nothing launched: on with the tokens themselves
                live, flight = [s for s in members if s.reason is None], None
                continue
            carried = [members[i] for i in going]
            with profiler.section(profiler.SAMPLING):
                if history is not None:                         # the tokens this step was fed count as seen from now on
                    history.mark_on_device([s.sampler.seen_row for s in carried], ids)
                picks = pick_batch(logits, [s.sampler for s in carried], history)
            for s in members:
                if s.reason is None:
                    settle(s)
            fed = [s for s in carried if s.reason is None]      # the others were carried a step too far
            for s in fed:
                s.sampler.history.append(s.next_token)
                s.generated += 1
            stats.decode_tokens += len(fed)
            stats.decode_steps += 1 if fed else 0
            flight = _Flight(carried, picks, pinned, stats.decode_steps & 1)
        stats.decode_seconds += time.perf_counter() - t0
    finally:
        for slot in held:
            cache.release(slot)
    return done


def generate(engine, prompts: Sequence[Sequence[int]], max_new_tokens: int = 600,
             sampling: SamplingParams | Sequence[SamplingParams] | None = None, stop_token_ids: Sequence[int] = (), ignore_eos: bool = False,
             max_batch: int | None = None, on_token=None) -> GenerationResult:
    """Generate for every prompt; results in the order of the prompts.  ``sampling``: one ``SamplingParams``
    for all of them, or a list with one per prompt."""
    sampling = sampling or SamplingParams()
    if not isinstance(sampling, SamplingParams):
        sampling = list(sampling)
        if len(sampling) != len(prompts):
            raise ShapeError(f"{len(sampling)} sampling parameters for {len(prompts)} prompts")
    if max_new_tokens < 1:
        raise ShapeError("max_new_tokens must be at least 1")
    cache = engine.cache
    total_pages = min((g.pool.num_pages for g in cache.groups), default=1 << 30)
    batches = plan_batches([len(p) for p in prompts], max_new_tokens, cache.page_size, total_pages,
                           cache.num_slots, cache.max_seq_len, max_batch)
    stats = GenerationStats()
    tokens, reasons = [None] * len(prompts), [None] * len(prompts)
    stop = frozenset(int(t) for t in stop_token_ids)
    for batch in batches:
        done = run_batch(engine, list(batch), prompts, max_new_tokens, sampling, stop, ignore_eos, stats, on_token)
        stats.batches += 1
        for r, (out, reason) in done.items():
            tokens[r], reasons[r] = out, reason
    return GenerationResult(tokens, reasons, stats)
