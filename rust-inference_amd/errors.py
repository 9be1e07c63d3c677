"""Error classes of the library: one per kind of failure a caller may want to tell apart.

They follow the variants of the reference's error type (src/error.rs:4-36): a bad or
unsupported configuration, a checkpoint that does not fit the model, a tensor of
the wrong shape, a cache that is full, a device or kernel problem.
"""


class InferenceError(Exception):
    """Base of every error this library raises on purpose."""


class ConfigError(InferenceError):
    """config.json is missing a key, holds an impossible value, or asks for something unsupported."""


class UnsupportedError(InferenceError):
    """An architecture, dtype or option that this library does not implement."""


class WeightsError(InferenceError):
    """The checkpoint does not match the model: lists missing, unexpected and misshapen tensors."""


class ShapeError(InferenceError):
    """An operand's shape or dtype is not what a kernel or part was built for."""


class CacheError(InferenceError):
    """The cache has no free slot or page, or a slot is used wrongly."""


class KernelError(InferenceError):
    """The HIP extension is missing, failed to build, or refused a launch."""
