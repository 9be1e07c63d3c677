"""Next-token selection on the host, stage by stage as the reference does it
(src/sampling.rs:73-128): repetition penalty, greedy if the temperature is not
positive, else temperature, top-k, sort by falling value (rising id among equals),
softmax, top-p prefix, one uniform draw.  The stages themselves are native host code
(csrc/plain/plain.cpp: ri_plain_sample); this is the per-sequence object around them."""
from __future__ import annotations

import numpy as np

from ..kernels import plain
from .params import SamplingParams
from .rng import Xorshift64Star


class HostSampler:
    """One sequence's sampler: its parameters and its own generator."""

    def __init__(self, params: SamplingParams, seed: int | None = None):
        self.params = params
        self.rng = Xorshift64Star(params.seed if seed is None else seed)

    def sample(self, logits, history=()) -> int:
        p = self.params
        return plain.sample(np.asarray(logits, dtype=np.float32), history, p.temperature, p.top_k, p.top_p,
                            p.repetition_penalty, self.rng)
