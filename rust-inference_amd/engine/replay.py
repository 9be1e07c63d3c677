"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and owns no model code: it reads one JSON object per line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

maps request ids to cache slots, calls the engine's step function, writes the
wanted logits of step N to ``<out>/N.f32`` (little-endian float32, ``[wanted, vocab]``,
in the order of the entries and of ``want``) and prints ``done N``.
"""
from __future__ import annotations

import json
import os
import sys

import torch

from ..cache import PAGE_SIZE
from ..errors import InferenceError
from ..parts import load_model
from .step import Engine, StepEntry


class Replayer:
    """Feeds trace steps to an engine, keeping the map from request ids to cache slots."""

    def __init__(self, engine: Engine):
        self.engine = engine
        self.slot_of: dict[str, int] = {}

    def feed(self, msg: dict):
        """Run one step; returns the float32 logits ``[wanted, vocab]`` on the device, or None
        when the step wants nothing."""
        cache = self.engine.cache
        entries = []
        for e in msg.get("entries", []):
            rid = str(e["id"])
            if rid not in self.slot_of:
                self.slot_of[rid] = cache.acquire()
            entries.append(StepEntry(self.slot_of[rid], e["tokens"], list(e.get("want", []))))
        logits = self.engine.step(entries) if entries else None
        for rid in msg.get("end", []):
            rid = str(rid)
            if rid not in self.slot_of:
                raise InferenceError(f"step {msg.get('step')} ends request {rid!r}, which never started")
            cache.release(self.slot_of.pop(rid))
        return logits if logits is not None and logits.shape[0] > 0 else None


def engine_for_trace(model, max_tokens: int) -> Engine:
    """An engine whose cache holds ``max_tokens`` tokens of live requests, each request's count
    rounded up to a multiple of 64 by the caller (whole pages, where a page divides 64; else the cache
    rounds every request up to its own pages, and the trace's bound is read as that many pages' worth)."""
    max_tokens = max(max_tokens, PAGE_SIZE)
    unit = max(64, PAGE_SIZE)                     # the smallest request the bound counts
    cache = model.new_cache(max_tokens=max_tokens, num_slots=max(1, -(-max_tokens // unit)),
                            max_seq_len=max_tokens)
    return Engine(model, cache)


def run(model_dir: str, dtype: torch.dtype, out_dir: str, max_tokens: int, lines=None, device="cuda:0",
        reply=None, invariant: bool = False) -> int:
    lines = sys.stdin if lines is None else lines
    reply = reply or (lambda s: print(s, flush=True))
    os.makedirs(out_dir, exist_ok=True)
    player = Replayer(engine_for_trace(load_model(model_dir, dtype, device, invariant), max_tokens))
    for line in lines:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        logits = player.feed(msg)
        if logits is not None:
            data = logits.detach().to("cpu", torch.float32).contiguous().numpy()
            tmp = os.path.join(out_dir, f".{step}.f32.tmp")
            data.astype("<f4").tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        else:
            torch.cuda.synchronize()
        reply(f"done {step}")
    return 0
