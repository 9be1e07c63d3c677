"""The sampler's generator: xorshift64* seeded through splitmix64 (src/sampling.rs:28-54)."""
from __future__ import annotations

_M = (1 << 64) - 1


class Xorshift64Star:
    def __init__(self, seed: int):
        z = (seed + 0x9E3779B97F4A7C15) & _M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
        self.state = (z ^ (z >> 31)) | 1            # never zero

    def next_u64(self) -> int:
        x = self.state
        x ^= x >> 12
        x ^= (x << 25) & _M
        x ^= x >> 27
        self.state = x
        return (x * 0x2545F4914F6CDD1D) & _M

    def next_f32(self) -> float:
        """Uniform in [0, 1): the top 24 bits over 2^24, exact in float32."""
        return (self.next_u64() >> 40) / float(1 << 24)
