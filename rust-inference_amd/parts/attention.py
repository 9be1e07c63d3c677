"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import math

import torch

from ..cache import KVNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import build_part, register_part
from .spec import PartSpec


# Up to this many sequences a decode step norms and rotates q and k inside the attention kernel (one
# launch less per layer); beyond it the many workgroups each repeating that work cost more than the
# launch (measured at 64 sequences of 2,048 tokens: 140 us against 111 + 6 us; at 24 and 32 sequences the
# one kernel is still ahead, by 1% of the step).  Steps that the attention takes with its streaming kernel
# (a workgroup per run of a sequence's pages: ops.decode_attention_streams) repeat little of it and are
# fused at any size.
FUSED_DECODE_MAX_SEQS = 32


@register_part("mixer", "attention")
class GroupedQueryAttention(Mixer):
    """q/k/v projections (no bias), optional per-head RMSNorm of q and k with one
    gain of ``head_dim`` shared by all heads, position encoding of q and k, write of
    k and v into the sequence's pages, causal attention of every new token over its
    sequence (all keys, or the last ``window``), output projection
    (the reference: src/models/qwen3.rs:71-100; src/attention.rs:33-150).

    Query head ``h`` reads kv head ``h // (heads / kv_heads)``; the score is
    ``(q . k) / sqrt(head_dim)``; softmax statistics and the accumulator are float32.
    The three projections are one product with the row-concatenated weight
    ``[q; k; v]``: every output row's dot product is the same as with three products.
    """

    links_norms = True

    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, prefix: str, qk_norm: bool = True,
                 eps: float = 1e-6, position: PartSpec | None = None, window: int | None = None):
        if heads < 1 or kv_heads < 1 or heads % kv_heads:
            raise ConfigError(f"{heads} attention heads not divisible by {kv_heads} kv heads")
        if head_dim % 16:
            raise ConfigError(f"head_dim {head_dim}: the attention kernels take multiples of 16")
        if window is not None and window < 1:
            raise ConfigError(f"window {window} must be positive")
        self.hidden, self.heads, self.kv_heads, self.head_dim = hidden, heads, kv_heads, head_dim
        self.prefix, self.qk_norm, self.eps, self.window = prefix, qk_norm, eps, window
        self.scale = 1.0 / math.sqrt(head_dim)                      # src/attention.rs:28
        self.position = build_part("position", position or PartSpec("none"))

    def tensors(self):
        p, d, dh = self.prefix, self.hidden, self.head_dim
        t = {
            p + "q_proj.weight": TensorSpec((self.heads * dh, d), MATRIX),
            p + "k_proj.weight": TensorSpec((self.kv_heads * dh, d), MATRIX),
            p + "v_proj.weight": TensorSpec((self.kv_heads * dh, d), MATRIX),
            p + "o_proj.weight": TensorSpec((d, self.heads * dh), MATRIX),
        }
        if self.qk_norm:
            t[p + "q_norm.weight"] = TensorSpec((dh,), GAIN)
            t[p + "k_norm.weight"] = TensorSpec((dh,), GAIN)
        t.update(self.position.tensors())
        return t

    def bind(self, weights, rt):
        self.rt = rt
        p = self.prefix
        qkv = torch.cat([weights[p + "q_proj.weight"], weights[p + "k_proj.weight"], weights[p + "v_proj.weight"]], 0)
        self.w_qkv = rt.pack(rt.place_matrix(qkv))
        self.w_o = rt.pack(rt.place_matrix(weights[p + "o_proj.weight"]))
        self.q_gain = rt.place_gain(weights[p + "q_norm.weight"]) if self.qk_norm else None
        self.k_gain = rt.place_gain(weights[p + "k_norm.weight"]) if self.qk_norm else None
        self.position.bind(weights, rt)

    def takes_tiled_at(self, m: int) -> bool:
        """Whether this part's first product reads ``m`` rows in the matrix cores' order."""
        return self.rt.takes_tiled(self.w_qkv, m)

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window)

    def forward(self, x, ctx, store, page_table, link=None):
        rt = self.rt
        qkv = rt.linear_packed(x, self.w_qkv)
        self.position.apply(qkv, ctx, self.heads, self.kv_heads, self.head_dim)
        group = self.heads // self.kv_heads
        if (ctx.is_decode and ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, True)
                and (ctx.B <= FUSED_DECODE_MAX_SEQS
                     or ops.decode_attention_streams(ctx.B, self.kv_heads, ctx.max_len))):
            # one token per sequence: norm, rotation, cache write and attention are one kernel
            o = ops.attention_decode_fused_bf16(qkv, self.q_gain, self.k_gain, self.eps,
                                                self.position.rotation_table(), store.k_pages, store.v_pages,
                                                ctx.tok_pos, page_table, ctx.B, ctx.max_len, self.heads,
                                                self.kv_heads, self.head_dim, self.window, self.scale,
                                                tiled_out=rt.takes_tiled(self.w_o, ctx.B))
            return rt.linear_packed(o, self.w_o, link=link)
        ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, self.eps, self.position.rotation_table(),
                                  ctx.tok_pos, ctx.tok_seq, page_table, store.k_pages, store.v_pages,
                                  self.heads, self.kv_heads, self.head_dim, ctx.cu_seqlens, ctx.max_new)
        return rt.linear_packed(self.attend(qkv, ctx, store, page_table), self.w_o, link=link)

    def attend(self, qkv, ctx, store, page_table):
        """The attention kernel that fits the step: matrix cores for bfloat16 (one new token per
        sequence, or any number), the generic kernel for everything else."""
        args = (self.heads, self.kv_heads, self.head_dim, self.window, self.scale)
        group = self.heads // self.kv_heads
        if ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, ctx.is_decode):
            if ctx.is_decode:
                return ops.attention_decode_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                                 page_table, ctx.B, ctx.max_len, *args,
                                                 tiled_out=self.rt.takes_tiled(self.w_o, ctx.B))
            return ops.attention_prefill_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                              page_table, ctx.B, ctx.max_new, *args)
        return ops.attention(qkv, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, *args)
