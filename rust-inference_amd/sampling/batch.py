"""Sampling for a batch: one generator and one history per sequence, so that a sequence's tokens do
not depend on what else is in its batch.  On the GPU the selection itself is the device kernel
(one workgroup per sequence); the uniform draws come from each sequence's host generator."""
from __future__ import annotations

import torch

from ..kernels import ops
from .host import HostSampler
from .params import SamplingParams


def upload(values, dtype, device) -> torch.Tensor:
    """A short list of numbers as a tensor on ``device`` without the host waiting for the GPU: through pinned
    memory, the copy in stream order (a copy from ordinary memory makes the host wait until everything launched
    before it is done, which is the step that the loop has just launched ahead)."""
    t = torch.tensor(values, dtype=dtype)
    device = torch.device(device)
    if device.type != "cuda":
        return t.to(device)
    return t.pin_memory().to(device, non_blocking=True)


class SequenceSampler:
    """The sampling state of one sequence.  Sequence ``index`` of a call draws from the generator
    seeded ``seed + index``; sequence 0 has the reference's stream."""

    def __init__(self, params: SamplingParams, index: int, prompt):
        self.params = params
        self.host = HostSampler(params, seed=(params.seed + index) & ((1 << 64) - 1))
        self.history = list(prompt)          # prompt plus generated, for the repetition penalty
        self.seen_row = None                 # this sequence's row of the device history, when there is one


class DeviceHistory:
    """The repetition penalty's history on the device: a byte per vocabulary entry and sequence."""

    def __init__(self, samplers: list[SequenceSampler], vocab: int, device):
        self.seen = torch.zeros((len(samplers), vocab), dtype=torch.uint8, device=device)
        rows, toks = [], []
        for r, s in enumerate(samplers):
            s.seen_row = r
            rows.extend([r] * len(s.history))
            toks.extend(s.history)
        self.mark(rows, toks)

    def mark_on_device(self, rows, tokens: torch.Tensor) -> None:
        """The same with the tokens still on the device (int32), so that nobody has to have read them."""
        if rows:
            ops.mark_seen(self.seen, upload(rows, torch.int32, self.seen.device), tokens)

    def mark(self, rows, tokens) -> None:
        if rows:
            dev = self.seen.device
            ops.mark_seen(self.seen, upload(rows, torch.int32, dev), upload(tokens, torch.int32, dev))


def _pick_alike(logits: torch.Tensor, samplers: list[SequenceSampler], history: DeviceHistory | None) -> torch.Tensor:
    """The rows of a batch whose sequences sample alike: one launch."""
    p = samplers[0].params
    if p.greedy and p.repetition_penalty == 1.0:
        return ops.argmax(logits)
    dev = logits.device
    uniform = None
    if not p.greedy:
        uniform = upload([s.host.rng.next_f32() for s in samplers], torch.float32, dev)
    seen = seen_rows = None
    if p.repetition_penalty != 1.0:
        if history is None:
            raise ValueError("a repetition penalty needs the device history of the batch")
        seen = history.seen
        seen_rows = upload([s.seen_row for s in samplers], torch.int32, dev)
    return ops.sample(logits, uniform, p.temperature, p.top_k, p.top_p, p.repetition_penalty, seen, seen_rows)


def _alike(p: SamplingParams) -> tuple:
    """What two sequences must share to be picked in one launch (each draws from its own generator anyway)."""
    return (max(p.temperature, 0.0), p.top_k, p.top_p, p.repetition_penalty)


def pick_batch(logits: torch.Tensor, samplers: list[SequenceSampler], history: DeviceHistory | None = None) -> torch.Tensor:
    """One token per row of float32 ``logits [B, vocab]`` as int32 ids where the logits are (on the GPU nothing
    waits for them); appends nothing to the histories.  Sequences may sample each in its own way: the rows are
    grouped by their parameters and every group is one launch (a batch that samples alike, the usual case, is one
    group and its logits are not copied)."""
    if logits.shape[0] != len(samplers):
        raise ValueError(f"{logits.shape[0]} rows of logits for {len(samplers)} sequences")
    if not logits.is_cuda:          # logits that never were on a GPU (tests of the loop): the host sampler
        rows = logits.detach().to(torch.float32).numpy()
        return torch.tensor([s.host.sample(rows[i], s.history) for i, s in enumerate(samplers)], dtype=torch.int32)
    groups: dict[tuple, list[int]] = {}
    for i, s in enumerate(samplers):
        groups.setdefault(_alike(s.params), []).append(i)
    if len(groups) == 1:
        return _pick_alike(logits, samplers, history)
    out = torch.empty(len(samplers), dtype=torch.int32, device=logits.device)
    for members in groups.values():
        at = upload(members, torch.int64, logits.device)
        out.index_copy_(0, at, _pick_alike(logits.index_select(0, at), [samplers[i] for i in members], history))
    return out


def sample_batch(logits: torch.Tensor, samplers: list[SequenceSampler], history: DeviceHistory | None = None) -> list[int]:
    """One token per row of float32 ``logits [B, vocab]``, read back to the host; appends nothing to the
    histories."""
    return pick_batch(logits, samplers, history).tolist()
