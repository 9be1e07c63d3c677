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

from ..errors import InferenceError
from ..parts import load_model
from .step import Engine, StepEntry


def run(model_dir: str, dtype: torch.dtype, out_dir: str, max_tokens: int, lines=None, device="cuda:0",
        reply=None) -> int:
    lines = sys.stdin if lines is None else lines
    reply = reply or (lambda s: print(s, flush=True))
    os.makedirs(out_dir, exist_ok=True)
    model = load_model(model_dir, dtype, device)
    page = 32
    # a request's count is rounded up to 64 by the caller: pages of 32 tokens fit inside that
    num_slots = max(1, -(-max_tokens // 64))
    cache = model.new_cache(max_tokens=max(max_tokens, page), num_slots=num_slots,
                            max_seq_len=min(max(max_tokens, page), model.spec.max_positions))
    engine = Engine(model, cache)
    slot_of: dict[str, int] = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        entries = []
        for e in msg.get("entries", []):
            rid = str(e["id"])
            if rid not in slot_of:
                slot_of[rid] = cache.acquire()
            entries.append(StepEntry(slot_of[rid], e["tokens"], list(e.get("want", []))))
        if entries:
            logits = engine.step(entries)
            if logits.shape[0] > 0:
                data = logits.detach().to("cpu", torch.float32).contiguous().numpy()
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                data.astype("<f4").tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
            else:
                torch.cuda.synchronize()
        for rid in msg.get("end", []):
            rid = str(rid)
            if rid not in slot_of:
                raise InferenceError(f"step {step} ends request {rid!r}, which never started")
            cache.release(slot_of.pop(rid))
        reply(f"done {step}")
    return 0
