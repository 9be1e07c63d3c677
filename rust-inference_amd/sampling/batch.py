"""Sampling for a batch: one generator and one history per sequence, so that a
sequence's tokens do not depend on what else is in its batch."""
from __future__ import annotations

import torch

from ..kernels import ops
from .host import HostSampler
from .params import SamplingParams


class SequenceSampler:
    """The sampling state of one sequence.  Sequence ``index`` of a call draws from the
    generator seeded ``seed + index``; sequence 0 has the reference's stream."""

    def __init__(self, params: SamplingParams, index: int, prompt):
        self.params = params
        self.host = HostSampler(params, seed=(params.seed + index) & ((1 << 64) - 1))
        self.history = list(prompt)          # prompt plus generated, for the repetition penalty


def sample_batch(logits: torch.Tensor, samplers: list[SequenceSampler]) -> list[int]:
    """One token per row of float32 ``logits [B, vocab]``; appends nothing to the histories."""
    if logits.shape[0] != len(samplers):
        raise ValueError(f"{logits.shape[0]} rows of logits for {len(samplers)} sequences")
    plain_greedy = all(s.params.greedy and s.params.repetition_penalty == 1.0 for s in samplers)
    if plain_greedy and logits.is_cuda:
        return ops.argmax(logits).tolist()
    rows = logits.detach().to("cpu", torch.float32).numpy()
    return [s.host.sample(rows[i], s.history) for i, s in enumerate(samplers)]
