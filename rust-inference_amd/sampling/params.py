"""Options of next-token selection, with the reference's names, defaults and meanings
(src/sampling.rs:9-26; command line: src/bin/runner.rs:78-96)."""
from __future__ import annotations

from dataclasses import dataclass

DEFAULT_SEED = 0x5EED


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0          # 0 (or less) means greedy
    top_k: int = 0                    # 0 disables top-k filtering
    top_p: float = 1.0                # 1.0 disables nucleus filtering
    repetition_penalty: float = 1.0   # 1.0 disables; positive logits are divided, others multiplied
    seed: int = DEFAULT_SEED

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0
