"""The generic decoder: embedding, layers in schedule order, final norm, output matrix.

Built from a ``ModelSpec``; which parts the layers have is the spec's business.
"""
from __future__ import annotations

import torch

from ..cache import Cache, KVNeed
from ..config import load_config
from ..errors import ConfigError, ShapeError
from .. import profiler
from ..kernels import ops
from ..weights.loader import MATRIX, TensorSpec, load_checked
from ..weights.random_init import random_tensors
from .base import Embedding, Head
from .block import ResidualStream
from .registry import build_part, part_class, register_part
from .runtime import Runtime
from .spec import ModelSpec


@register_part("embedding", "table")
class TokenEmbedding(Embedding):
    """``h[t, :] = E[id_t, :]`` without scaling (the reference: src/ops/embedding.rs:10-42)."""

    def __init__(self, vocab: int, dim: int, name: str):
        self.vocab, self.dim, self.name = vocab, dim, name

    def tensors(self):
        return {self.name: TensorSpec((self.vocab, self.dim), MATRIX)}

    def bind(self, weights, rt):
        self.rt = rt
        self.table = rt.place_matrix(weights[self.name])

    def forward(self, ctx):
        return ops.embed_gather(self.table, ctx.tokens)

    def bind_plain(self, weights):
        self.table_plain = weights[self.name].to(torch.float32).numpy()

    def plain(self, ctx):
        from ..kernels import plain
        return plain.embedding(self.table_plain, ctx.tokens)


@register_part("head", "linear")
class OutputHead(Head):
    """``logits = x W^T`` in float32, no scaling or cap.  The matrix is the embedding
    table when the configuration ties them or the checkpoint has no tensor of this
    name (the reference: src/models/qwen3.rs:167-171, :286)."""

    def __init__(self, vocab: int, dim: int, name: str, tied: bool):
        self.vocab, self.dim, self.name, self.tied = vocab, dim, name, tied

    def tensors(self):
        return {self.name: TensorSpec((self.vocab, self.dim), MATRIX, optional=True)}

    def written_when_random(self) -> bool:
        return not self.tied

    def bind(self, weights, rt):
        self.rt = rt
        self.weight = self.packed = None
        if not self.tied and self.name in weights:
            self.weight = rt.place_matrix(weights[self.name])

    def connect(self, parts):
        if self.weight is None:
            table = getattr(parts.get("embedding"), "table", None)
            if table is None or tuple(table.shape) != (self.vocab, self.dim):
                raise ConfigError(f"{self.name} is absent and there is no embedding table of {self.vocab} x {self.dim} "
                                  "to tie it to")
            self.weight = table                     # the same device tensor: tying costs no memory

    def bind_plain(self, weights):
        self.weight_plain = None
        if not self.tied and self.name in weights:
            self.weight_plain = weights[self.name].to(torch.float32).numpy()

    def connect_plain(self, parts):
        if self.weight_plain is None:
            self.weight_plain = getattr(parts.get("embedding"), "table_plain", None)
            if self.weight_plain is None or self.weight_plain.shape != (self.vocab, self.dim):
                raise ConfigError(f"{self.name} is absent and there is no embedding table to tie it to")

    def plain(self, x):
        from ..kernels import plain
        return plain.linear(x, self.weight_plain)

    def _packed_copy(self):
        """A second copy of the matrix in the matrix cores' tile order, for steps that want 2 to 32 or 48 rows of
        logits (a decode step of as many sequences): at 151,936 x 4,096 the packed kernel takes 0.21 ms where
        the library's product takes 0.26 (1% of such a step), for 1.2 GB more memory.  It is made at the first
        such step, so that a model which never runs one (a single slot, or only larger batches) does not pay
        for it; never while a graph is being captured (the engine runs every step once before it captures it)."""
        if self.packed is None and not torch.cuda.is_current_stream_capturing():
            self.packed = self.rt.pack(self.weight, always=True)
        return self.packed

    # Rows of logits up to which the packed copy serves: 2 to 8 the packed kernel (one load of x serves two steps of
    # K there); from 9 on the wide kernel with four row tiles a workgroup, which shares the rows of x through LDS
    # (151,936 x 4,096 at 9, 16, 17 and 32 rows: 204, 213, 222 and 247 us against the packed kernel's 224 and 279
    # and the library's 250 to 279; x 1,024 at 16 rows 57 against 78; x 5,120: 254 against 382; from 48 rows on the
    # library is ahead, 266 against 279 us, with 39 MB of float32 logits to write).  33 to 48 rows with three tiles of
    # x, for rows of up to 4,096 elements: eight layers and this matrix at 33 / 40 / 47 sequences are 1.5 / 1.5 / 0.9%
    # shorter at Qwen3-0.6B sizes, 3.7 / 2.8 / 1.8% at 4B, 1.2 / 0.8 / 0% at 8B; with rows of 5,120 (32B) 0 to 0.7% longer.
    PACKED_MAX_ROWS = 32
    PACKED_MORE_ROWS = 48            # for rows of up to PACKED_MORE_DIM elements
    PACKED_MORE_DIM = 4096
    PAIRED_MAX_ROWS = 8

    def forward(self, x):
        rows = x.shape[0]
        if self.rt.invariant:
            return self.rt.linear_packed(x, self._packed_copy(), out_dtype=torch.float32)
        most = self.PACKED_MORE_ROWS if self.dim <= self.PACKED_MORE_DIM else self.PACKED_MAX_ROWS
        if 2 <= rows <= most and self.dim % 8 == 0:
            packed = self._packed_copy()
            if packed is not None and packed.packed is not None:
                if rows <= self.PAIRED_MAX_ROWS:
                    return self.rt.linear_packed(x, packed, out_dtype=torch.float32)
                return ops.gemm_wide_packed_bf16(self.rt.normed_now(x), packed.packed, self.vocab, torch.float32,
                                                 depth=1, waves=4)
        return self.rt.linear(x, self.weight, out_dtype=torch.float32)


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.layers = [part_class("arrangement", ls.arrangement)(ls) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.schedule = list(spec.schedule)
        for r in self.schedule:
            if not 0 <= r.layer < len(self.layers):
                raise ConfigError(f"schedule names layer {r.layer}, the model has {len(self.layers)}")
        self.rt = None

    # ---- weights
    def parts(self):
        yield self.embedding
        for layer in self.layers:
            yield from layer.parts()
        yield self.final_norm
        yield self.head

    def tensors(self, for_writing: bool = False) -> dict[str, TensorSpec]:
        out = {}
        for part in self.parts():
            if for_writing and part is self.head and not self.head.written_when_random():
                continue
            for name, spec in part.tensors().items():
                if name in out and out[name].shape != spec.shape:
                    raise ConfigError(f"tensor {name} is wanted with shapes {out[name].shape} and {spec.shape}")
                out[name] = spec
        return out

    def bind(self, weights: dict, rt: Runtime) -> "DecoderModel":
        self.rt = rt
        self.embedding.bind(weights, rt)
        for layer in self.layers:
            for part in layer.parts():
                part.bind(weights, rt)
        self.final_norm.bind(weights, rt)
        self.head.bind(weights, rt)
        named = {"embedding": self.embedding, "layers": self.layers, "final_norm": self.final_norm, "head": self.head}
        for part in self.parts():
            connect = getattr(part, "connect", None)
            if connect is not None:
                connect(named)
        return self

    def bind_plain(self, weights: dict) -> "DecoderModel":
        """Take the weights for the plain backend: every part keeps float32 numpy arrays.  A part that has no
        plain form is named in the error."""
        for part in self.parts():
            if not hasattr(part, "bind_plain") or not hasattr(part, "plain"):
                raise ConfigError(f"the part {type(part).__name__} has no plain form: the CPU backend cannot run this model")
        for layer in self.layers:
            if not hasattr(layer, "plain"):
                raise ConfigError(f"the arrangement {type(layer).__name__} has no plain form")
        for part in self.parts():
            part.bind_plain(weights)
        named = {"embedding": self.embedding, "layers": self.layers, "final_norm": self.final_norm, "head": self.head}
        for part in self.parts():
            if hasattr(part, "connect_plain"):
                part.connect_plain(named)
        return self

    def plain_forward(self, ctx, stores, page_tables):
        """float32 logits ``[n_want, vocab]`` (numpy) of a step on the CPU: ``stores[entry]`` is the cache entry's
        storage (a pair of page arrays), ``page_tables[group]`` the step's table of its group."""
        h = self.embedding.plain(ctx)
        for run in self.schedule:
            entries = run.entries()
            if len(entries) != 1:
                raise ConfigError("the plain backend runs layers with one cache entry")
            store, group = stores[entries[0]]
            h = self.layers[run.layer].plain(h, ctx, store, page_tables[group])
        return self.head.plain(self.final_norm.plain(h[ctx.want_rows]))

    # ---- cache
    def cache_needs(self) -> list:
        """The need of every cache entry the schedule names.  A layer says what it keeps per sequence
        through its arrangement's ``cache_need()`` (by default its mixer's): one need, or a tuple of
        them for a run that names a tuple of entries."""
        needs = [None] * self.spec.num_cache_entries
        for r in self.schedule:
            entries = r.entries()
            if not entries:
                continue
            layer = self.layers[r.layer]
            asked = layer.cache_need() if hasattr(layer, "cache_need") else layer.mixer.cache_need()
            asked = tuple(asked) if isinstance(asked, (tuple, list)) else (asked,)
            if len(asked) != len(entries):
                raise ConfigError(f"layer {r.layer} keeps {len(asked)} things per sequence, its run names "
                                  f"{len(entries)} cache entries")
            for entry, need in zip(entries, asked):
                if needs[entry] is not None and needs[entry] != need:
                    raise ConfigError(f"cache entry {entry} is used with two different needs")
                needs[entry] = need
        return needs

    def new_cache(self, max_tokens: int, num_slots: int, max_seq_len: int | None = None, **kw) -> Cache:
        # the configuration's max_position_embeddings is the default length only: nothing in this
        # architecture depends on it (the reference reads it and never uses it, src/models/config.rs:30)
        max_seq_len = max_seq_len or self.spec.max_positions
        return Cache(self.cache_needs(), num_slots, max_tokens, max_seq_len, dtype=self.rt.dtype,
                     device=self.rt.device, **kw)

    # ---- one step
    def forward(self, ctx, cache: Cache) -> torch.Tensor:
        """float32 logits ``[n_want, vocab]`` for the wanted rows of this step's tokens."""
        rt = self.rt
        with profiler.section(profiler.EMBEDDING):
            stream = ResidualStream(self.embedding.forward(ctx))
        stream.links_ok = not rt.invariant
        for at, run in enumerate(self.schedule):
            layer = self.layers[run.layer]
            follower = self.layers[self.schedule[at + 1].layer] if at + 1 < len(self.schedule) else None
            entry = getattr(follower, "entry_norm", None)
            stream.next_entry_norm = entry() if entry else None
            tiled = getattr(follower, "entry_takes_tiled", None)
            stream.next_entry_tiled = tiled(stream.sum.shape[0]) if tiled else False
            stores, tables = [], []
            for entry in run.entries():
                need = cache.needs[entry]
                if isinstance(need, KVNeed):
                    stores.append(cache.kv(entry))
                    tables.append(ctx.page_tables[stores[-1].group_index])
                else:
                    stores.append(cache.state(entry) if need is not None else None)
                    tables.append(None)
            if isinstance(run.cache, (tuple, list)):          # a layer with several entries gets them all, in order
                store, table = tuple(stores), tuple(tables)
            else:
                store, table = (stores[0], tables[0]) if stores else (None, None)
            layer.forward(stream, ctx, store, table, rt.dtype)
        if ctx.n_want == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=rt.device)
        h = stream.normed(self.final_norm, rt.dtype, rows=ctx.want_rows)      # only the wanted rows
        with profiler.section(profiler.LM_HEAD):
            logits = self.head.forward(h)
        if logits.shape != (ctx.n_want, self.spec.vocab_size):
            raise ShapeError(f"logits are {list(logits.shape)}")
        return logits


def expected_tensors(spec: ModelSpec, for_writing: bool = False) -> dict[str, TensorSpec]:
    return DecoderModel(spec).tensors(for_writing)


def load_model(model_dir: str, dtype=torch.bfloat16, device="cuda:0", invariant: bool = False) -> DecoderModel:
    """The model of a folder: the class by config.json, the weights by name.  ``invariant``: see ``Runtime``."""
    arch, cfg = load_config(model_dir)
    model = DecoderModel(arch.build_spec(cfg))
    model.config = cfg
    weights = load_checked(model_dir, model.tensors())
    return model.bind(weights, Runtime(device, dtype, invariant))


def load_model_plain(model_dir: str) -> DecoderModel:
    """The model of a folder for the CPU backend: the same class and the same checks, the weights kept as
    float32 numpy arrays by the parts' plain forms."""
    arch, cfg = load_config(model_dir)
    model = DecoderModel(arch.build_spec(cfg))
    model.config = cfg
    return model.bind_plain(load_checked(model_dir, model.tensors()))


def random_model(config, seed: int, dtype=torch.bfloat16, device="cuda:0", store_dtype=torch.bfloat16,
                 invariant: bool = False) -> DecoderModel:
    """A model with random weights made in memory, for sizes one would not write to disk."""
    from ..config import config_from_dict
    arch, cfg = config_from_dict(config if isinstance(config, dict) else config.to_dict())
    model = DecoderModel(arch.build_spec(cfg))
    model.config = cfg
    rt = Runtime(device, dtype, invariant)
    weights = random_tensors(model.tensors(for_writing=True), seed, store_dtype, device=rt.device)
    return model.bind(weights, rt)
