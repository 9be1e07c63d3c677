from .batch import DeviceHistory, SequenceSampler, pick_batch, sample_batch
from .host import HostSampler
from .params import DEFAULT_SEED, SamplingParams
from .rng import Xorshift64Star

__all__ = ["DeviceHistory", "SequenceSampler", "pick_batch", "sample_batch", "HostSampler", "SamplingParams", "DEFAULT_SEED", "Xorshift64Star"]
