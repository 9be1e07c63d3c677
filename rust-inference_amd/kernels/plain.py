"""Python face of the plain C++ twins of the kernels (csrc/plain): float32 numpy arrays in and out.

Host code only; nothing here touches a GPU.  The tests hold these functions against the float64
implementation under tests/plain, and the kernels are checked against both; `sample` and the generator are
also what `sampling.HostSampler` runs on."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_float, c_int, c_int32, c_uint16, c_uint64, c_void_p

import numpy as np

from ..errors import ShapeError
from .build import load_plain

_lib = None


def lib():
    global _lib
    if _lib is None:
        l = load_plain()
        l.ri_plain_f32_to_bf16.argtypes, l.ri_plain_f32_to_bf16.restype = [c_float], c_uint16
        l.ri_plain_bf16_to_f32.argtypes, l.ri_plain_bf16_to_f32.restype = [c_uint16], c_float
        l.ri_plain_embedding.argtypes, l.ri_plain_embedding.restype = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int], c_int
        l.ri_plain_rms_norm.argtypes, l.ri_plain_rms_norm.restype = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_float], None
        l.ri_plain_add_rms_norm.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float]
        l.ri_plain_add_rms_norm.restype = None
        l.ri_plain_rope_inv_freq.argtypes, l.ri_plain_rope_inv_freq.restype = [c_void_p, c_int, c_float], None
        l.ri_plain_rope.argtypes, l.ri_plain_rope.restype = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int], None
        l.ri_plain_linear.argtypes, l.ri_plain_linear.restype = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int], None
        l.ri_plain_swiglu.argtypes, l.ri_plain_swiglu.restype = [c_void_p, c_void_p, c_int, c_int], None
        l.ri_plain_attention.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                         c_int, c_int, c_int, c_int, c_int, c_float]
        l.ri_plain_attention.restype = None
        l.ri_plain_argmax.argtypes, l.ri_plain_argmax.restype = [c_void_p, c_int], c_int
        l.ri_plain_rng_seed.argtypes, l.ri_plain_rng_seed.restype = [c_uint64], c_uint64
        l.ri_plain_rng_next.argtypes, l.ri_plain_rng_next.restype = [POINTER(c_uint64)], c_uint64
        l.ri_plain_rng_next_f32.argtypes, l.ri_plain_rng_next_f32.restype = [POINTER(c_uint64)], c_float
        l.ri_plain_sample.argtypes = [c_void_p, c_int, c_void_p, c_int, c_float, c_int, c_float, c_float, POINTER(c_uint64)]
        l.ri_plain_sample.restype = c_int
        _lib = l
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


def f32_to_bf16(f: float) -> int:
    return lib().ri_plain_f32_to_bf16(float(f))


def bf16_to_f32(b: int) -> float:
    return lib().ri_plain_bf16_to_f32(int(b))


def embedding(table, ids) -> np.ndarray:
    table, ids = _f32(table), _i32(ids)
    out = np.empty((ids.shape[0], table.shape[1]), dtype=np.float32)
    if lib().ri_plain_embedding(_p(out), _p(table), _p(ids), ids.shape[0], table.shape[0], table.shape[1]):
        raise ShapeError(f"token id out of range for a table of {table.shape[0]} rows")
    return out


def rms_norm(x, gain, eps: float) -> np.ndarray:
    """Over the last axis (whose length is the gain's: a per-head norm is the same call on ``[..., head_dim]``)."""
    x, gain = _f32(x), _f32(gain)
    out = np.empty_like(x)
    lib().ri_plain_rms_norm(_p(out), _p(x), _p(gain), x.size // gain.shape[0], gain.shape[0], float(eps))
    return out


def add_rms_norm(residual, pending, gain, eps: float):
    """``(residual + pending, norm of it)``."""
    residual, pending, gain = _f32(residual).copy(), _f32(pending), _f32(gain)
    out = np.empty_like(residual)
    lib().ri_plain_add_rms_norm(_p(out), _p(residual), _p(pending), _p(gain), residual.size // gain.shape[0],
                                gain.shape[0], float(eps))
    return residual, out


def rope_inv_freq(rot_dim: int, theta: float) -> np.ndarray:
    out = np.empty(rot_dim // 2, dtype=np.float32)
    lib().ri_plain_rope_inv_freq(_p(out), int(rot_dim), float(np.float32(theta)))
    return out


def rope(x, positions, inv_freq) -> np.ndarray:
    """Rotate-half on ``x: [tokens, heads, head_dim]`` over the first ``2 * len(inv_freq)`` elements of each head."""
    x, positions, inv_freq = _f32(x).copy(), _i32(positions), _f32(inv_freq)
    tokens, heads, head_dim = x.shape
    lib().ri_plain_rope(_p(x), _p(positions), _p(inv_freq), tokens, heads, head_dim, 2 * inv_freq.shape[0])
    return x


def linear(x, w) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    if x.shape[1] != w.shape[1]:
        raise ShapeError(f"linear: x has {x.shape[1]} columns, the weight {w.shape[1]}")
    out = np.empty((x.shape[0], w.shape[0]), dtype=np.float32)
    lib().ri_plain_linear(_p(out), _p(x), _p(w), x.shape[0], w.shape[0], x.shape[1])
    return out


def swiglu(y) -> np.ndarray:
    y = _f32(y)
    out = np.empty((y.shape[0], y.shape[1] // 2), dtype=np.float32)
    lib().ri_plain_swiglu(_p(out), _p(y), y.shape[0], y.shape[1] // 2)
    return out


def attention(q, k_pages, v_pages, tok_pos, tok_seq, page_table, window: int | None, scale: float) -> np.ndarray:
    """``q: [tokens, heads, head_dim]`` over pages ``k: [pages, kv_heads, page, head_dim]``, ``v: [pages, kv_heads,
    head_dim, page]``."""
    q, k_pages, v_pages = _f32(q), _f32(k_pages), _f32(v_pages)
    tok_pos, tok_seq, page_table = _i32(tok_pos), _i32(tok_seq), _i32(page_table)
    tokens, heads, head_dim = q.shape
    _, kv_heads, page_size, dh = k_pages.shape
    if dh != head_dim or v_pages.shape != (k_pages.shape[0], kv_heads, head_dim, page_size) or heads % kv_heads:
        raise ShapeError(f"pages {k_pages.shape} / {v_pages.shape} do not fit queries {q.shape}")
    out = np.empty_like(q)
    lib().ri_plain_attention(_p(out), _p(q), _p(k_pages), _p(v_pages), _p(tok_pos), _p(tok_seq), _p(page_table),
                             page_table.shape[1], tokens, heads, kv_heads, head_dim, page_size, int(window or 0),
                             float(scale))
    return out


def argmax(row) -> int:
    row = _f32(row)
    return lib().ri_plain_argmax(_p(row), row.shape[0])


class Rng:
    """The sampler's generator (src/sampling.rs:33-53) with its state on the native side's terms."""

    def __init__(self, seed: int):
        self._state = c_uint64(lib().ri_plain_rng_seed(seed & ((1 << 64) - 1)))

    @property
    def state(self) -> int:
        return self._state.value

    def next_u64(self) -> int:
        return lib().ri_plain_rng_next(ctypes.byref(self._state))

    def next_f32(self) -> float:
        return lib().ri_plain_rng_next_f32(ctypes.byref(self._state))


def sample(logits, history, temperature: float, top_k: int, top_p: float, penalty: float, rng: Rng) -> int:
    logits, history = _f32(logits), _i32(history if len(history) else [])
    return lib().ri_plain_sample(_p(logits), logits.shape[0], _p(history), history.shape[0], float(temperature), int(top_k),
                                 float(top_p), float(penalty), ctypes.byref(rng._state))
