"""The layout of a step in plain numpy: what the cache's native writer (csrc/host_cache.hip:
ri_cache_plan_step) has to put into the block of words that goes to the device.  A test oracle; the
engine does not use it."""
import itertools

import numpy as np

from rust_inference_amd.engine import wanted_indices
from rust_inference_amd.errors import ShapeError


def plan_step(entries, lengths, vocab_size: int):
    """The host-side layout of a step: flat tokens, each token's sequence and position, where
    each sequence starts among them, and the wanted rows, as int32 arrays.  ``lengths[i]`` is
    entry i's cache length before the step."""
    if not entries:
        raise ShapeError("a step needs at least one entry")
    counts = [len(e.tokens) for e in entries]
    for b, (e, n) in enumerate(zip(entries, counts)):
        if n < 1:
            raise ShapeError(f"entry {b} (slot {e.slot}) brings no token")
    total = sum(counts)
    tokens = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int64, count=total)
    if tokens.min() < 0 or tokens.max() >= vocab_size:
        bad = int(tokens[(tokens < 0) | (tokens >= vocab_size)][0])
        raise ShapeError(f"token id {bad} is outside the vocabulary of {vocab_size}")       # src/ops/embedding.rs:20-22
    cu = np.zeros(len(entries) + 1, dtype=np.int32)
    np.cumsum(counts, out=cu[1:])
    if total == len(entries):                                  # one token each: the common step
        tok_seq = np.arange(total, dtype=np.int32)
        tok_pos = np.asarray(lengths, dtype=np.int32)
    else:
        tok_seq = np.repeat(np.arange(len(entries), dtype=np.int32), counts)
        tok_pos = (np.arange(total, dtype=np.int32) - np.repeat(cu[:-1] - np.asarray(lengths, dtype=np.int32), counts))
    want_rows = np.asarray([int(cu[b]) + i for b, (e, n) in enumerate(zip(entries, counts))
                            for i in wanted_indices(n, e.want)], dtype=np.int32)
    return tokens.astype(np.int32), tok_seq, tok_pos.astype(np.int32), cu, want_rows
