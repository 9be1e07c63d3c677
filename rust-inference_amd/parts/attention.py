"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import math

import torch

from .. import profiler
from ..cache import KVNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import build_part, register_part
from .spec import PartSpec


# Up to this many sequences a decode step norms and rotates q and k inside the attention kernel (one launch
# less per layer); beyond it the many workgroups each repeating that work are taken to cost more than the launch
# (up to 56 sequences of 8 kv heads they do not: 1 to 2.4% of the step).  Steps that the attention takes with its
# streaming kernel repeat little of it and are fused at any size.
FUSED_DECODE_MAX_SEQS = 64


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

    ``qkv_bias`` and ``o_bias`` add ``{q,k,v}_proj.bias`` and ``o_proj.bias`` to the products (the
    reference's family has no bias anywhere, src/models/qwen3.rs:60-69; families that differ from it in
    this alone need no other mixer).  A biased output product adds into the stream the plain way.
    """

    links_norms = True

    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, prefix: str, qk_norm: bool = True,
                 eps: float = 1e-6, position: PartSpec | None = None, window: int | None = None,
                 qkv_bias: bool = False, o_bias: bool = False):
        if heads < 1 or kv_heads < 1 or heads % kv_heads:
            raise ConfigError(f"{heads} attention heads not divisible by {kv_heads} kv heads")
        if not 1 <= head_dim <= ops.MAX_HEAD_DIM:
            raise ConfigError(f"head_dim {head_dim}: the attention kernels take 1 to {ops.MAX_HEAD_DIM}")
        if window is not None and window < 1:
            raise ConfigError(f"window {window} must be positive")
        self.hidden, self.heads, self.kv_heads, self.head_dim = hidden, heads, kv_heads, head_dim
        self.prefix, self.qk_norm, self.eps, self.window = prefix, qk_norm, eps, window
        self.qkv_bias, self.o_bias = qkv_bias, o_bias
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
        if self.qkv_bias:
            t[p + "q_proj.bias"] = TensorSpec((self.heads * dh,), BIAS)
            t[p + "k_proj.bias"] = TensorSpec((self.kv_heads * dh,), BIAS)
            t[p + "v_proj.bias"] = TensorSpec((self.kv_heads * dh,), BIAS)
        if self.o_bias:
            t[p + "o_proj.bias"] = TensorSpec((d,), BIAS)
        t.update(self.position.tensors())
        return t

    def bind(self, weights, rt):
        self.rt = rt
        p = self.prefix
        qkv = torch.cat([weights[p + "q_proj.weight"], weights[p + "k_proj.weight"], weights[p + "v_proj.weight"]], 0)
        self.w_qkv = rt.pack(rt.place_matrix(qkv))
        self.w_o = rt.pack(rt.place_matrix(weights[p + "o_proj.weight"]), parts_ok=(p + "o_proj.bias") not in weights)
        self.q_gain = rt.place_gain(weights[p + "q_norm.weight"]) if self.qk_norm else None
        self.k_gain = rt.place_gain(weights[p + "k_norm.weight"]) if self.qk_norm else None
        self.b_qkv = self.b_o = None
        if self.qkv_bias:
            self.b_qkv = rt.place_gain(torch.cat([weights[p + n + "_proj.bias"] for n in "qkv"], 0))
        if self.o_bias:
            self.b_o = rt.place_gain(weights[p + "o_proj.bias"])
        self.position.bind(weights, rt)

    def bind_plain(self, weights):
        f32 = lambda name: weights[self.prefix + name].to(torch.float32).numpy()
        self.plain_w = {n: f32(n + "_proj.weight") for n in "qkvo"}
        self.plain_gain = {n: f32(n + "_norm.weight") for n in "qk"} if self.qk_norm else {}
        self.plain_bias = {n: f32(n + "_proj.bias") for n in ("qkv" if self.qkv_bias else "") + ("o" if self.o_bias else "")}
        if getattr(self.position, "acts_after_norm", False) or not hasattr(self.position, "plain"):
            raise ConfigError(f"the position encoding {type(self.position).__name__} has no plain form")
        self.position.bind_plain(weights)

    def plain(self, x, ctx, store, page_table):
        """The same over numpy arrays and the plain C++ twins: three products, per-head norm, rotation, the new keys
        and values into their pages (``store = (k_pages, v_pages)``, values transposed inside a page), attention
        over the pages, output product."""
        from ..kernels import plain
        t, dh, page = x.shape[0], self.head_dim, store[0].shape[2]
        heads = {}
        for n, count in (("q", self.heads), ("k", self.kv_heads), ("v", self.kv_heads)):
            y = plain.linear(x, self.plain_w[n])
            if n in self.plain_bias:
                y = y + self.plain_bias[n]
            heads[n] = y.reshape(t, count, dh)
        for n in "qk":
            if self.qk_norm:
                heads[n] = plain.rms_norm(heads[n], self.plain_gain[n], self.eps)
            heads[n] = self.position.plain(heads[n], ctx.tok_pos)
        phys = page_table[ctx.tok_seq, ctx.tok_pos // page]
        store[0][phys, :, ctx.tok_pos % page, :] = heads["k"]
        store[1][phys, :, :, ctx.tok_pos % page] = heads["v"]
        o = plain.attention(heads["q"], store[0], store[1], ctx.tok_pos, ctx.tok_seq, page_table, self.window, self.scale)
        y = plain.linear(o.reshape(t, self.heads * dh), self.plain_w["o"])
        return y + self.plain_bias["o"] if "o" in self.plain_bias else y

    def takes_tiled_at(self, m: int) -> bool:
        """Whether this part's first product reads ``m`` rows in the matrix cores' order."""
        return self.rt.takes_tiled(self.w_qkv, m)

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window)

    def forward(self, x, ctx, store, page_table, link=None):
        rt = self.rt
        with profiler.section(profiler.QKV_PROJECTION):
            qkv = rt.linear_packed(x, self.w_qkv)
            if self.b_qkv is not None:
                ops.add_bias(qkv, self.b_qkv)
        self.position.apply(qkv, ctx, self.heads, self.kv_heads, self.head_dim)
        group = self.heads // self.kv_heads
        table = self.position.rotation_table()
        whole = table is None or 2 * table.shape[0] == self.head_dim      # the fused kernel rotates whole heads
        after_norm = getattr(self.position, "acts_after_norm", False)
        if (ctx.is_decode and whole and not after_norm and not rt.invariant
                and ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, True)
                and (ctx.B <= FUSED_DECODE_MAX_SEQS
                     or ops.decode_attention_streams(ctx.B, self.kv_heads, ctx.max_len))):
            # one token per sequence: norm, rotation, cache write and attention are one kernel
            with profiler.section(profiler.ATTENTION):
                o = ops.attention_decode_fused_bf16(qkv, self.q_gain, self.k_gain, self.eps, table, store.k_pages,
                                                    store.v_pages, ctx.tok_pos, page_table, ctx.B, ctx.max_len,
                                                    self.heads, self.kv_heads, self.head_dim, self.window, self.scale,
                                                    tiled_out=rt.takes_tiled(self.w_o, ctx.B, self.b_o is None))
            return self.project_out(o, link)
        with profiler.section(profiler.QK_NORM_ROPE_APPEND):
            shape = (self.heads, self.kv_heads, self.head_dim)
            if after_norm:
                # an encoding that acts on the normed q and k: norm (and rotation) in place, the encoding,
                # then the move of k and v into their pages
                ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, self.eps, table, ctx.tok_pos, ctx.tok_seq,
                                          page_table, None, None, *shape)
                self.position.apply_normed(qkv, ctx, *shape)
                ops.qk_norm_rope_kv_write(qkv, None, None, self.eps, None, ctx.tok_pos, ctx.tok_seq, page_table,
                                          store.k_pages, store.v_pages, *shape, ctx.cu_seqlens, ctx.max_new)
            elif rt.invariant:
                # the kernel of one wavefront per token and head, whatever the step looks like
                ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, self.eps, table, ctx.tok_pos, ctx.tok_seq,
                                          page_table, store.k_pages, store.v_pages, *shape)
            else:
                ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, self.eps, table, ctx.tok_pos, ctx.tok_seq,
                                          page_table, store.k_pages, store.v_pages, *shape, ctx.cu_seqlens, ctx.max_new)
        with profiler.section(profiler.ATTENTION):
            o = self.attend(qkv, ctx, store, page_table)
        return self.project_out(o, link)

    def project_out(self, o, link):
        with profiler.section(profiler.OUT_PROJECTION):
            if self.b_o is None:
                return self.rt.linear_packed(o, self.w_o, parts_ok=True, link=link)
            return ops.add_bias(self.rt.linear_packed(o, self.w_o), self.b_o)

    def attend(self, qkv, ctx, store, page_table):
        """The attention kernel that fits the step: matrix cores for bfloat16 (one new token per
        sequence, or any number), the generic kernel for everything else."""
        args = (self.heads, self.kv_heads, self.head_dim, self.window, self.scale)
        group = self.heads // self.kv_heads
        if self.rt.invariant:
            # one kernel for prompts and single tokens alike: in the prompt kernel a token's sums run over its
            # sequence's pages in order whatever the other rows of its tile are (a page that a row does not
            # see changes none of its bits); the generic kernel where that one does not take the sizes
            if ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, False):
                return ops.attention_prefill_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                                  page_table, ctx.B, ctx.max_new, *args)
            return ops.attention(qkv, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, *args)
        if ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, ctx.is_decode):
            if ctx.is_decode:
                return ops.attention_decode_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                                 page_table, ctx.B, ctx.max_len, *args,
                                                 tiled_out=self.rt.takes_tiled(self.w_o, ctx.B, self.b_o is None))
            return ops.attention_prefill_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                              page_table, ctx.B, ctx.max_new, *args)
        return ops.attention(qkv, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, *args)
