"""Next-token selection on the host, stage by stage as the reference does it
(src/sampling.rs:73-128): repetition penalty, greedy if the temperature is not
positive, else temperature, top-k, sort by falling value (rising id among equals),
softmax, top-p prefix, one uniform draw."""
from __future__ import annotations

import numpy as np

from .params import SamplingParams
from .rng import Xorshift64Star


def apply_repetition_penalty(row: np.ndarray, history, penalty: float) -> np.ndarray:
    if penalty == 1.0 or not len(history):
        return row
    row = row.copy()
    seen = np.unique(np.asarray(history, dtype=np.int64))
    seen = seen[(seen >= 0) & (seen < row.shape[0])]
    vals = row[seen]
    row[seen] = np.where(vals > 0, vals / np.float32(penalty), vals * np.float32(penalty))
    return row


def first_argmax(row: np.ndarray) -> int:
    return int(np.argmax(row))          # numpy returns the first of equal maxima


def kept_candidates(row: np.ndarray, p: SamplingParams):
    """Token ids in drawing order and their float32 probabilities."""
    scaled = (row / np.float32(p.temperature)).astype(np.float32)
    order = np.lexsort((np.arange(scaled.shape[0]), -scaled))      # value falling, id rising among equals
    if 0 < p.top_k < order.shape[0]:
        order = order[:p.top_k]
    vals = scaled[order]
    probs = np.exp(vals - vals[0], dtype=np.float32)
    probs = probs / probs.sum(dtype=np.float32)
    if p.top_p < 1.0:
        acc = np.cumsum(probs, dtype=np.float32)
        reach = np.nonzero(acc >= np.float32(p.top_p))[0]
        keep = int(reach[0]) + 1 if reach.size else probs.shape[0]
        probs = probs[:keep]
        probs = probs / probs.sum(dtype=np.float32)
        order = order[:keep]
    return order, probs


class HostSampler:
    """One sequence's sampler: its parameters and its own generator."""

    def __init__(self, params: SamplingParams, seed: int | None = None):
        self.params = params
        self.rng = Xorshift64Star(params.seed if seed is None else seed)

    def sample(self, logits, history=()) -> int:
        p = self.params
        row = apply_repetition_penalty(np.asarray(logits, dtype=np.float32), history, p.repetition_penalty)
        if p.greedy:
            return first_argmax(row)
        order, probs = kept_candidates(row, p)
        r = np.float32(self.rng.next_f32())
        acc = np.cumsum(probs, dtype=np.float32)
        hit = np.nonzero(r < acc)[0]
        return int(order[int(hit[0])] if hit.size else order[probs.shape[0] - 1])
