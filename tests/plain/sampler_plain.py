"""Plain next-token selection, written from src/sampling.rs of the reference.

One function per stage so that the engine's device sampler can be compared with it
stage by stage.  32-bit arithmetic where the reference uses it.
"""
from __future__ import annotations

import numpy as np

MASK64 = (1 << 64) - 1


class PlainRng:
    """xorshift64* seeded through the splitmix64 finaliser (src/sampling.rs:33-48);
    ``next_f32`` is the top 24 bits over 2^24, in [0, 1) (src/sampling.rs:51-53)."""

    def __init__(self, seed: int):
        z = (seed + 0x9E3779B97F4A7C15) & MASK64
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
        self.state = (z ^ (z >> 31)) | 1

    def next_u64(self) -> int:
        x = self.state
        x ^= x >> 12
        x = (x ^ (x << 25)) & MASK64
        x ^= x >> 27
        self.state = x
        return (x * 0x2545F4914F6CDD1D) & MASK64

    def next_f32(self) -> float:
        return float(np.float32(self.next_u64() >> 40) / np.float32(1 << 24))


def penalise(logits: np.ndarray, history, penalty: float) -> np.ndarray:
    """Every token id present in the history: a positive logit is divided by the
    penalty, any other multiplied (src/sampling.rs:76-88)."""
    out = np.array(logits, dtype=np.float32)
    if penalty != 1.0:
        for t in set(int(t) for t in history):
            if 0 <= t < len(out):
                out[t] = out[t] / np.float32(penalty) if out[t] > 0 else out[t] * np.float32(penalty)
    return out


def argmax(row) -> int:
    """First index of the maximum (src/sampling.rs:131-139)."""
    best = 0
    for i in range(len(row)):
        if row[i] > row[best]:
            best = i
    return best


def candidates(logits: np.ndarray, temperature: float, top_k: int, top_p: float):
    """The kept token ids in drawing order and their probabilities: divide by the
    temperature, keep the k largest, sort by falling value and rising id, softmax
    with the maximum subtracted, keep the shortest prefix whose mass reaches top_p
    and normalise again (src/sampling.rs:93-117)."""
    scaled = (np.asarray(logits, dtype=np.float32) / np.float32(temperature)).astype(np.float32)
    order = sorted(range(len(scaled)), key=lambda i: (-float(scaled[i]), i))
    if 0 < top_k < len(order):
        order = order[:top_k]
    vals = scaled[order]
    probs = np.exp((vals - vals[0]).astype(np.float32)).astype(np.float32)
    probs = (probs / probs.sum(dtype=np.float32)).astype(np.float32)
    if top_p < 1.0:
        acc, keep = np.float32(0.0), len(probs)
        for i, q in enumerate(probs):
            acc = np.float32(acc + q)
            if acc >= np.float32(top_p):
                keep = i + 1
                break
        probs = probs[:keep]
        probs = (probs / probs.sum(dtype=np.float32)).astype(np.float32)
        order = order[:keep]
    return order, probs


def draw(order, probs, r: float) -> int:
    """The first candidate whose running sum exceeds ``r``; the last kept one if none
    does (src/sampling.rs:119-127)."""
    acc = np.float32(0.0)
    for tok, q in zip(order, probs):
        acc = np.float32(acc + q)
        if r < acc:
            return int(tok)
    return int(order[len(probs) - 1])


class PlainSampler:
    """src/sampling.rs:56-128 as one object: penalty, then greedy if the temperature
    is not positive, else the filtered draw with this sampler's own generator."""

    def __init__(self, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0, seed=0x5EED):
        self.temperature, self.top_k, self.top_p = temperature, top_k, top_p
        self.repetition_penalty = repetition_penalty
        self.rng = PlainRng(seed)

    def sample(self, logits, history=()) -> int:
        row = penalise(logits, history, self.repetition_penalty)
        if self.temperature <= 0.0:
            return argmax(row)
        order, probs = candidates(row, self.temperature, self.top_k, self.top_p)
        return draw(order, probs, self.rng.next_f32())
