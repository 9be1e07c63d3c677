"""The Python entry point: load a model folder, generate, or step by hand.

It mirrors the reference's library demo (examples/generate.rs:12-44: load, make
caches, loop {forward, pick, stop?, append}) with its runner's option names
(src/bin/runner.rs:24-123), for batches of prompts given as token ids.
"""
from __future__ import annotations

import math
from typing import Sequence

import torch

from .cache import PAGE_SIZE
from .engine import Engine, GenerationResult, StepEntry, generate as _generate
from .engine.plain_engine import PlainEngine
from .parts import load_model, load_model_plain, random_model
from .sampling import DEFAULT_SEED, SamplingParams

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           "f32": torch.float32}


def as_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        return dtype
    try:
        return _DTYPES[str(dtype).lower()]
    except KeyError:
        raise ValueError(f"dtype {dtype!r}: expected bfloat16 or float32") from None


# A graph of a batch size is worth capturing at once where launching a step's kernels from the host takes as long as
# the step: a small model.  Where the step's weights take longer to read than its kernels to launch, host launches
# cost a few per cent and the capture what several steps take, so a size that lives for a step or two is better left
# without one.  The two times are estimated from what is known before any step has run: the weights' bytes at 5 TB/s,
# and seven launches a layer at 8 us.  Measured through generate(), ms for the whole call, capture at the first step :
# after the third: 200 prompts whose sequences stop at random steps (a hundred batch sizes) on three layers of
# Qwen3-14B sizes 365 : 268, on Qwen3-0.6B 642 : 693; 64 prompts on twelve layers of Qwen3-8B sizes 655 : 578, 16
# prompts there 316 : 308, 16 prompts on Qwen3-0.6B 541 : 545.
_WEIGHTS_BYTES_PER_SECOND = 5e12
_LAUNCH_SECONDS, _LAUNCHES_PER_LAYER = 8e-6, 7
_DEFERRED_CAPTURE = 3


def capture_after_for(decoder) -> int:
    """How many steps of a batch size should run with host launches before their graph is captured, for this model."""
    try:
        width = 2 if decoder.rt.dtype == torch.bfloat16 else 4
        elements = sum(math.prod(spec.shape) for spec in decoder.tensors().values())
        layers = len(decoder.schedule)
    except Exception:
        return 0
    reading = elements * width / _WEIGHTS_BYTES_PER_SECOND
    launching = layers * _LAUNCHES_PER_LAYER * _LAUNCH_SECONDS
    return _DEFERRED_CAPTURE if reading > launching else 0


class Model:
    """A loaded model with a cache sized for ``max_batch`` sequences of ``max_seq_len`` tokens.
    ``graph_after``: decode steps of one batch size run that many times with host launches before their graph is
    captured (capturing costs 3 to 5 steps' time, and a batch whose sequences stop at different times passes
    through many sizes); 0 captures at the first step of a size; None, the default, chooses by the model's size
    (``capture_after_for``)."""

    def __init__(self, decoder, max_batch: int = 8, max_seq_len: int = 4096, max_tokens: int | None = None,
                 use_graphs: bool = True, plain: bool = False, graph_after: int | None = None):
        self.decoder = decoder
        self.config = getattr(decoder, "config", None)
        per_seq = -(-max_seq_len // PAGE_SIZE) * PAGE_SIZE
        if plain:
            self.engine = PlainEngine(decoder, max_batch, max_tokens or per_seq * max_batch, max_seq_len)
            self.cache = self.engine.cache
        else:
            self.cache = decoder.new_cache(max_tokens or per_seq * max_batch, max_batch, max_seq_len)
            if graph_after is None:
                graph_after = capture_after_for(decoder) if use_graphs else 0
            self.engine = Engine(decoder, self.cache, use_graphs=use_graphs, capture_after=graph_after)

    @classmethod
    def load(cls, model_dir: str, dtype="bfloat16", device="cuda:0", batch_invariant: bool = False,
             **cache_options) -> "Model":
        """``batch_invariant`` (bfloat16 on the GPU): every step runs the same form of every kernel, so that a
        request's logits and tokens are the same bits in any batch and any cut (``parts.runtime.Runtime``).
        ``device="cpu"`` chooses the plain backend (the reference's ``--device cpu``, src/bin/runner.rs:98-100):
        the whole model in float32 on the scalar C++ twins of the kernels, for the parts that have a plain form."""
        if str(device).startswith("cpu"):
            if as_dtype(dtype) != torch.float32:
                raise ValueError("the CPU backend computes in float32 (weights stay as stored and are widened exactly)")
            return cls(load_model_plain(model_dir), plain=True, **cache_options)
        return cls(load_model(model_dir, as_dtype(dtype), device, batch_invariant), **cache_options)

    @classmethod
    def random(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0", batch_invariant: bool = False,
               **cache_options) -> "Model":
        """Random weights made in memory from a config.json dict or a typed configuration."""
        return cls(random_model(config, seed, as_dtype(dtype), device, invariant=batch_invariant), **cache_options)

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 600, temperature: float = 0.0,
                 top_k: int = 0, top_p: float = 1.0, repetition_penalty: float = 1.0, seed: int = DEFAULT_SEED,
                 stop_token_ids: Sequence[int] = (), ignore_eos: bool = False, max_batch: int | None = None,
                 on_token=None, sampling: Sequence[SamplingParams] | None = None) -> GenerationResult:
        """The options are the reference runner's (src/bin/runner.rs:78-96) and hold for every prompt;
        ``sampling`` instead gives every prompt its own ``SamplingParams``."""
        params = sampling if sampling is not None else SamplingParams(temperature, top_k, top_p, repetition_penalty, seed)
        return _generate(self.engine, prompts, max_new_tokens, params, stop_token_ids, ignore_eos, max_batch, on_token)

    def step(self, entries) -> torch.Tensor:
        """``entries``: ``(slot, tokens, want)`` triples; float32 logits at the wanted places."""
        return self.engine.step([e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries])


def generate(model_dir: str, prompts, dtype="bfloat16", **options) -> list:
    """One call from a folder to generated token ids."""
    longest = max(len(p) for p in prompts) + options.get("max_new_tokens", 600)
    model = Model.load(model_dir, dtype, max_batch=min(len(prompts), 64), max_seq_len=longest)
    return model.generate(prompts, **options).tokens
