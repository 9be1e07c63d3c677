"""The sampler's generator: xorshift64* seeded through splitmix64 (src/sampling.rs:28-54).  The generator
itself is native host code (csrc/plain/plain.cpp); ``next_f32`` is uniform in [0, 1): the top 24 bits over
2^24, exact in float32."""
from __future__ import annotations

from ..kernels.plain import Rng


class Xorshift64Star(Rng):
    pass
