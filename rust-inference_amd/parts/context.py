"""What one step looks like to the parts: the flattened tokens of all sequences and
where each belongs."""
from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass
class StepContext:
    """All new tokens of a step, sequence after sequence: ``T`` tokens of ``B``
    sequences.  Positions come from the cache lengths, never from the caller (the
    reference takes positions and cache lengths as separate inputs that must agree:
    src/models/qwen3.rs:275-278 against src/attention.rs:73).

    Device tensors (int32): ``tokens [T]``, ``tok_seq [T]`` (index of the token's
    sequence in this step), ``tok_pos [T]`` (its absolute position), ``cu_seqlens
    [B + 1]``, ``slots [B]``, ``len_after [B]``, ``want_rows [n_want]`` (flat token
    indices whose logits are asked for), and one ``page_tables[g] [B, width]`` per
    key/value group of the cache.  The same as Python lists on the host side.
    """
    T: int
    B: int
    new_counts: list
    slot_list: list
    starts: list                     # length of each sequence before this step
    tokens: torch.Tensor = None
    tok_seq: torch.Tensor = None
    tok_pos: torch.Tensor = None
    cu_seqlens: torch.Tensor = None
    slots: torch.Tensor = None
    len_after: torch.Tensor = None
    want_rows: torch.Tensor = None
    n_want: int = 0
    page_tables: list = field(default_factory=list)
    max_new: int = 0                 # most new tokens of any sequence
    max_len: int = 0                 # longest sequence after this step

    @property
    def is_decode(self) -> bool:
        return self.max_new == 1
