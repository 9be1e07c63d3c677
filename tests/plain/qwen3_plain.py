"""Plain, slow, whole-sequence implementation of the Qwen3 dense decoder.

Written from the formulas of thanhauco/rust-inference; every function cites the
file and lines it was read from (paths relative to the reference's root).  It
works on whole sequences in float64 numpy, keeps no cache, has one function per
part, and shares no code with the engine: the engine is compared against it.

Weights are a dict from the checkpoint's tensor names to float64 arrays.
"""
from __future__ import annotations

import numpy as np


# --------------------------------------------------------------------------- parts

def embedding(table: np.ndarray, ids) -> np.ndarray:
    """Row gather ``h[t, :] = E[id_t, :]``; an id outside the table is an error
    (src/ops/embedding.rs:10-42, ids checked at :15-22)."""
    ids = np.asarray(ids, dtype=np.int64)
    if ids.size and (ids.min() < 0 or ids.max() >= table.shape[0]):
        raise ValueError(f"token id out of range for a table of {table.shape[0]} rows")
    return table[ids]


def rms_norm(x: np.ndarray, gain: np.ndarray, eps: float) -> np.ndarray:
    """``y_i = x_i * (1 / sqrt(mean_j(x_j^2) + eps)) * w_i`` over the last axis:
    eps sits inside the root and the gain multiplies directly, not as ``1 + w``
    (src/ops/norm.rs:7-10 for the scale, :25-30 for the product)."""
    ss = np.mean(x * x, axis=-1, keepdims=True)
    return x * (1.0 / np.sqrt(ss + eps)) * gain


def rope_inv_freq(head_dim: int, theta: float) -> np.ndarray:
    """``inv_freq[i] = 1 / theta^(2i / head_dim)`` for ``i < head_dim / 2``, computed in
    32-bit: theta itself is a 32-bit number (src/models/config.rs:33-34) and so are
    the exponent and the power (src/ops/rope.rs:20)."""
    i = np.arange(head_dim // 2, dtype=np.float32)
    expo = (np.float32(2.0) * i) / np.float32(head_dim)
    return (np.float32(1.0) / np.power(np.float32(theta), expo, dtype=np.float32)).astype(np.float32)


def rope_angles(positions, head_dim: int, theta: float) -> np.ndarray:
    """Angle ``f32(pos) * inv_freq[i]`` as a 32-bit product (src/ops/rope.rs:39); the
    sine and cosine are then taken of that 32-bit angle
    (scripts/reference_qwen3.py:119-124 keeps the 32-bit angle and widens after)."""
    pos = np.asarray(positions).astype(np.float32)
    ang = (pos[:, None] * rope_inv_freq(head_dim, theta)[None, :]).astype(np.float32)
    return ang.astype(np.float64)  # [S, head_dim / 2]


def apply_rope(x: np.ndarray, angles: np.ndarray) -> np.ndarray:
    """Rotate-half on ``x: [S, heads, head_dim]``: the pairs are ``(d, d + head_dim/2)``,
    ``x'[d] = x[d] cos - x[d+half] sin`` and ``x'[d+half] = x[d+half] cos + x[d] sin``
    (src/ops/rope.rs:73-74; both table halves hold the same angle, :40-43)."""
    half = x.shape[-1] // 2
    cos = np.cos(angles)[:, None, :]
    sin = np.sin(angles)[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return np.concatenate([x1 * cos - x2 * sin, x2 * cos + x1 * sin], axis=-1)


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, q_positions=None, window: int | None = None) -> np.ndarray:
    """Causal grouped-query attention of ``q: [S, H, dh]`` over ``k, v: [L, Hkv, dh]``.

    Query head ``h`` reads key/value head ``h // (H / Hkv)`` (src/attention.rs:4-6,
    :57-66).  The score is ``(q . k_j) * (1 / sqrt(dh))``: the scale multiplies the
    dot product (src/attention.rs:28, :121-127).  The query at absolute position
    ``p`` sees keys ``0..=p`` (src/attention.rs:73, :117-118); by default the
    queries are the last ``S`` of the ``L`` positions.  Softmax over the visible
    keys, then the weighted sum of values (src/attention.rs:128-149).

    ``window`` is not in the reference (all its layers see every key): with a window
    ``w`` the query at ``p`` sees keys ``max(0, p - w + 1)..=p``.  It is here for the
    tests of the engine's windowed cache group only.
    """
    s, h, dh = q.shape
    l, hkv, _ = k.shape
    group = h // hkv
    if q_positions is None:
        q_positions = np.arange(l - s, l)
    scale = 1.0 / np.sqrt(float(dh))
    out = np.zeros_like(q)
    for t in range(s):
        p = int(q_positions[t])
        lo = 0 if window is None else max(0, p - window + 1)
        for head in range(h):
            kv = head // group
            scores = (k[lo:p + 1, kv, :] @ q[t, head, :]) * scale
            e = np.exp(scores - scores.max())
            out[t, head, :] = (e / e.sum()) @ v[lo:p + 1, kv, :]
    return out


def silu(x: np.ndarray) -> np.ndarray:
    """``silu(z) = z / (1 + exp(-z))`` (src/ops/elementwise.rs:9-12)."""
    return x / (1.0 + np.exp(-x))


def swiglu_mlp(x: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray) -> np.ndarray:
    """``down(silu(gate(x)) * up(x))`` with ``y = x W^T`` and no bias anywhere
    (src/models/qwen3.rs:112-117; src/ops/linear.rs:7-19)."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def attention_block(x, w, prefix, cfg, positions, window=None):
    """q/k/v projections, per-head RMSNorm of q and k (one gain of ``head_dim`` shared
    by all heads, before the rotation, never on v), rotation of q and k, attention,
    output projection (src/models/qwen3.rs:82-99)."""
    s = x.shape[0]
    h, hkv, dh = cfg["num_attention_heads"], cfg["num_key_value_heads"], head_dim(cfg)
    eps = cfg.get("rms_norm_eps", 1e-6)
    q = (x @ w[prefix + "q_proj.weight"].T).reshape(s, h, dh)
    k = (x @ w[prefix + "k_proj.weight"].T).reshape(s, hkv, dh)
    v = (x @ w[prefix + "v_proj.weight"].T).reshape(s, hkv, dh)
    q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
    ang = rope_angles(positions, dh, cfg.get("rope_theta", 1e6))
    q, k = apply_rope(q, ang), apply_rope(k, ang)
    o = attention(q, k, v, window=window).reshape(s, h * dh)
    return o @ w[prefix + "o_proj.weight"].T


def decoder_layer(hid, w, i, cfg):
    """Pre-norm layer: ``r = h + attn(norm(h))`` is the new residual stream, then
    ``h' = r + mlp(norm(r))`` (src/models/qwen3.rs:130-144)."""
    p = f"model.layers.{i}."
    eps = cfg.get("rms_norm_eps", 1e-6)
    positions = np.arange(hid.shape[0])
    x = rms_norm(hid, w[p + "input_layernorm.weight"], eps)
    r = hid + attention_block(x, w, p + "self_attn.", cfg, positions)
    x = rms_norm(r, w[p + "post_attention_layernorm.weight"], eps)
    return r + swiglu_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])


# --------------------------------------------------------------------------- whole model

def head_dim(cfg) -> int:
    """``head_dim`` is a key of its own and falls back to ``hidden / heads``
    (src/models/config.rs:75-77)."""
    hd = cfg.get("head_dim")
    return int(hd) if hd else cfg["hidden_size"] // cfg["num_attention_heads"]


def lm_head_weight(cfg, w):
    """The output matrix is the embedding when the config ties them or when the file
    has no ``lm_head.weight`` (src/models/qwen3.rs:167-171)."""
    if cfg.get("tie_word_embeddings", False) or "lm_head.weight" not in w:
        return w["model.embed_tokens.weight"]
    return w["lm_head.weight"]


def forward(cfg: dict, w: dict, ids) -> np.ndarray:
    """Logits ``[S, V]`` of one whole sequence starting at position 0: embedding, the
    layers in order, final norm, output matrix (src/models/qwen3.rs:274-286)."""
    hid = embedding(w["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        hid = decoder_layer(hid, w, i, cfg)
    hid = rms_norm(hid, w["model.norm.weight"], cfg.get("rms_norm_eps", 1e-6))
    return hid @ lm_head_weight(cfg, w).T


def greedy(cfg: dict, w: dict, prompt, steps: int, stop_ids=()):
    """Greedy continuation by recomputing the whole sequence for every new token; the
    first of equal maxima wins (src/sampling.rs:131-139).  A stop token ends the
    sequence and is not part of the output (src/bin/runner.rs:293-295).  Returns
    the tokens and the logits each was chosen from."""
    ids, out, rows = list(prompt), [], []
    for _ in range(steps):
        row = forward(cfg, w, ids)[-1]
        nxt = argmax(row)
        rows.append(row)
        if nxt in stop_ids:
            break
        out.append(nxt)
        ids.append(nxt)
    return out, rows


def argmax(row) -> int:
    """Index of the first maximum (strict ``>``; src/ops/reduce.rs:18-25)."""
    best = 0
    for i in range(len(row)):
        if row[i] > row[best]:
            best = i
    return best


# --------------------------------------------------------------------------- numbers

def bf16_round(a: np.ndarray) -> np.ndarray:
    """Round 32-bit floats to bfloat16 and back: nearest, ties to even
    (src/dtype.rs:82-89)."""
    return bf16_bits_to_f32(f32_to_bf16_bits(a))


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    rounded = np.where(nan, (bits >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """A bfloat16 is the upper half of a 32-bit float (src/dtype.rs:75-77)."""
    return (bits.astype(np.uint32) << 16).view(np.float32)
