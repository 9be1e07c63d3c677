"""Section timers: device time per kind of work, off by default (the reference: src/profiler.rs:14-135).

``enable(True)`` (the runner's ``--profile``) turns them on; parts wrap their kernels in
``with section(NAME):``, which records a pair of events on the current stream around them, and
``report()`` prints the reference's table (section, total seconds, share, calls; largest first).  The
times are the GPU's own, taken from the events, not the host's.  While the timers are on, decode steps are
launched kernel by kernel instead of replayed as a graph (a captured graph holds no events to read), so a
profiled run is slower than an unprofiled one; shares stay meaningful.

The section names are the reference's where the work is the same (src/profiler.rs:52-69).  Where this
library runs several of the reference's sections as one kernel, the time is booked under the section whose
work dominates it: the decode attention kernel also norms and rotates q and k and appends to the cache
("attention"), and in small decode steps the norms run inside the products around them (no "rmsnorm" row).
"""
from __future__ import annotations

import torch

EMBEDDING = "embedding"
QKV_PROJECTION = "attn q/k/v proj"
QK_NORM_ROPE_APPEND = "attn q/k norm, rope, kv append"
ATTENTION = "attention"
OUT_PROJECTION = "attn o proj"
NORM = "rmsnorm"
MLP = "dense mlp"
LM_HEAD = "lm head"
SAMPLING = "sampling"

_enabled = False
_seconds: dict[str, float] = {}
_calls: dict[str, int] = {}
_open: list = []                     # (name, start event, end event) not yet read
_spare: list = []                    # events to use again
MAX_OPEN = 4096                      # pairs kept before they are read (reading waits for the GPU)


def enable(on: bool) -> None:
    global _enabled
    if not on:
        collect()
    _enabled = bool(on)


def enabled() -> bool:
    return _enabled


def reset() -> None:
    collect()
    _seconds.clear()
    _calls.clear()


class _Off:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_OFF = _Off()


class _Section:
    __slots__ = ("name", "start", "end")

    def __init__(self, name: str):
        self.name = name

    def __enter__(self):
        self.start = _spare.pop() if _spare else torch.cuda.Event(enable_timing=True)
        self.end = _spare.pop() if _spare else torch.cuda.Event(enable_timing=True)
        self.start.record()
        return self

    def __exit__(self, exc_type, *exc):
        self.end.record()
        if exc_type is None:
            _open.append((self.name, self.start, self.end))
            if len(_open) >= MAX_OPEN:
                collect()
        return False


def section(name: str):
    """A context manager that books the device time of what runs inside it to ``name`` (nothing when the
    timers are off, or while a graph is being captured)."""
    if not _enabled or torch.cuda.is_current_stream_capturing():
        return _OFF
    return _Section(name)


def collect() -> None:
    """Read the events recorded so far (waits for the GPU to reach the last of them)."""
    if not _open:
        return
    _open[-1][2].synchronize()
    for name, start, end in _open:
        _seconds[name] = _seconds.get(name, 0.0) + start.elapsed_time(end) * 1e-3
        _calls[name] = _calls.get(name, 0) + 1
        _spare.extend((start, end))
    _open.clear()


def snapshot() -> list[tuple[str, float, int]]:
    """``(section, total seconds, calls)`` for every section that ran."""
    collect()
    return [(name, _seconds[name], _calls[name]) for name in _seconds if _calls[name] > 0]


def report() -> str:
    """The breakdown, largest first, in the reference's layout (src/profiler.rs:113-123)."""
    rows = sorted(snapshot(), key=lambda r: -r[1])
    total = sum(r[1] for r in rows)
    out = ["section                          total(s)   share    calls"]
    for name, secs, calls in rows:
        share = 100.0 * secs / total if total > 0 else 0.0
        out.append(f"{name:<30} {secs:>10.4f} {share:>6.1f}% {calls:>8}")
    return "\n".join(out) + "\n"
