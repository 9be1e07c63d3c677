"""Python face of the HIP kernels: one function per kernel.

Each wrapper checks on the host that the operands are what the kernel and its
grid assume (device, dtype, contiguity, shapes) and then launches on torch's
current stream.  There is no other implementation behind these functions: without
the library, or on a tensor that is not on the GPU, they raise.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p

import torch

from ..errors import KernelError, ShapeError
from .build import load

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

_SIGNATURES = {
    "ri_embed_gather": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "ri_add_rmsnorm": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_int,
                       c_int, c_int, c_void_p],
    "ri_add_rows": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "ri_qk_norm_rope_kv_write": [c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int, c_void_p, c_void_p,
                                 c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_int, c_void_p],
    "ri_attention": [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                     c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "ri_attention_prefill_bf16": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                  c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "ri_attention_decode_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "ri_attention_decode_fused_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float,
                                       c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                       c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "ri_gemm_f32": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gemv_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ri_sample": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int, c_float, c_float,
                  c_void_p],
    "ri_mark_seen": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "ri_sample_split": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int,
                        c_float, c_float, c_void_p],
    "ri_gemm_skinny_packed_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gemm_mid_packed_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gemm_wide_packed_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_int, c_void_p],
    "ri_gemm_wide_packed_bf16_plan": [c_int, c_int, c_int, c_void_p, c_void_p],
    "ri_gemm_wide_stretch_plan": [c_int, c_int, c_int, c_void_p, c_void_p],
    "ri_compute_units": [],
    "ri_sum_parts": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_attention_decode_chunks": [c_int],
    "ri_attention_decode_streams": [c_int, c_int, c_int],
    "ri_attention_decode_pieces": [c_int, c_int, c_int, c_int],
    "ri_gemv_bf16_partials": [c_int, c_int],
    "ri_gemm_skinny_packed_bf16_partials": [c_int],
    "ri_gemv_bf16_linked": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float,
                            c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "ri_gemm_skinny_packed_bf16_linked": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p,
                                          c_int, c_float, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    "ri_swiglu": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ri_add_bias": [c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "ri_finish_norm": [c_void_p, c_void_p, c_void_p, c_int, c_float, c_int, c_int, c_int, c_void_p],
    "ri_argmax": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
}

_fn = {}


def _get(name: str):
    f = _fn.get(name)
    if f is None:
        lib = load()
        try:
            f = getattr(lib, name)
        except AttributeError:
            raise KernelError(f"the kernel library has no {name}: it is older than this package, build it again") from None
        f.argtypes = _SIGNATURES[name]
        f.restype = c_int
        _fn[name] = f
    return f


def _call(name: str, *args) -> None:
    rc = _get(name)(*args)
    if rc != 0:
        raise KernelError(load().ri_last_error().decode())


def _stream() -> int:
    """The current device's current stream, as the raw handle the kernels are launched on (torch's
    ``current_stream()`` builds a Python object through several layers for the same number: 5 us a call)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise ShapeError(f"dtype {dtype} is not float32 or bfloat16") from None


def _dev(t: torch.Tensor, name: str, dtype=None, shape=None) -> int:
    """Checks a tensor and returns its device address."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: the kernels run on the GPU only, got "
                          f"{t.device if isinstance(t, torch.Tensor) else type(t).__name__}")
    if not t.is_contiguous():
        raise ShapeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise ShapeError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ShapeError(f"{name} must have shape {list(shape)}, got {list(t.shape)}")
    return t.data_ptr()


def _opt(t, name: str, dtype=None, shape=None):
    return None if t is None else _dev(t, name, dtype, shape)


# ---------------------------------------------------------------- row-wise
def embed_gather(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """float32 rows ``table[ids]``; ids int32 ``[T]``, already checked to be inside the table."""
    tokens, dim = ids.shape[0], table.shape[1]
    out = torch.empty((tokens, dim), dtype=torch.float32, device=table.device)
    _call("ri_embed_gather", _dev(out, "out"), _dev(table, "table"), code(table.dtype),
          _dev(ids, "ids", torch.int32, (tokens,)), tokens, dim, _stream())
    return out


def add_rmsnorm(residual: torch.Tensor, pending, gain: torch.Tensor, eps: float, out_dtype,
                rows: torch.Tensor | None = None, tiled: bool = False):
    """``residual += pending`` (in place, when ``rows`` is None) and the RMSNorm of the sum.
    With ``rows`` the sum and norm are taken of those rows only and nothing is written back.
    ``pending`` may be ``[parts, T, dim]``: the parts of a product split along K, added in order.
    With ``tiled`` the normed rows (bfloat16, at most 64) come as ``TiledRows``."""
    t, dim = residual.shape
    n = t if rows is None else rows.shape[0]
    parts = 1
    if pending is not None and pending.dim() == 3:
        parts = pending.shape[0]
        if tuple(pending.shape[1:]) != (t, dim):
            raise ShapeError(f"pending parts are {list(pending.shape)}, the stream is {[t, dim]}")
    elif pending is not None and tuple(pending.shape) != (t, dim):
        raise ShapeError(f"pending is {list(pending.shape)}, the stream is {[t, dim]}")
    out = TiledRows.empty(n, dim, residual.device) if tiled else torch.empty((n, dim), dtype=out_dtype,
                                                                             device=residual.device)
    _call("ri_add_rmsnorm", _dev(out.data if tiled else out, "out"), code(out_dtype),
          _dev(residual, "residual", torch.float32),
          _opt(pending, "pending"), code(pending.dtype) if pending is not None else F32, parts, t,
          _dev(gain, "gain", torch.float32, (dim,)), float(eps), _opt(rows, "rows", torch.int32), n, dim, int(tiled),
          _stream())
    return out


def add_rows(residual: torch.Tensor, pending, rows: torch.Tensor | None = None, in_place: bool = False) -> torch.Tensor:
    """float32 ``residual[rows] + pending[rows]`` without a norm; with ``in_place`` (all rows) the sum is
    written into ``residual`` itself."""
    t, dim = residual.shape
    n = t if rows is None else rows.shape[0]
    if in_place and rows is not None:
        raise ShapeError("an add in place takes all rows")
    out = residual if in_place else torch.empty((n, dim), dtype=torch.float32, device=residual.device)
    _call("ri_add_rows", _dev(out, "out"), _dev(residual, "residual", torch.float32),
          _opt(pending, "pending", None, (t, dim)), code(pending.dtype) if pending is not None else F32,
          _opt(rows, "rows", torch.int32), n, dim, _stream())
    return out


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``x[t, :] += bias`` in place (float32 bias, the sum in float32); returns ``x``."""
    rows, dim = x.shape
    _call("ri_add_bias", _dev(x, "x"), code(x.dtype), _dev(bias, "bias", torch.float32, (dim,)), rows, dim, _stream())
    return x


def swiglu(y: torch.Tensor, tiled_out: bool = False):
    """``silu(y[:, :I]) * y[:, I:]`` for ``y: [T, 2 I]``; ``tiled_out``: the bfloat16 result as ``TiledRows``
    (at most 64 rows, ``I`` a multiple of 8)."""
    tokens, two_i = y.shape
    if two_i % 2:
        raise ShapeError(f"swiglu input has an odd width {two_i}")
    inter = two_i // 2
    tiled_out = tiled_out and y.dtype == torch.bfloat16 and tokens <= 64 and inter % 8 == 0
    out = TiledRows.empty(tokens, inter, y.device) if tiled_out else torch.empty((tokens, inter), dtype=y.dtype,
                                                                                   device=y.device)
    _call("ri_swiglu", _dev(out.data if tiled_out else out, "out"), _dev(y, "y"), code(y.dtype), tokens, inter,
          int(tiled_out), _stream())
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """int32 index of the first maximum of every row of float32 ``logits``."""
    rows, vocab = logits.shape
    ids = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    ws = torch.empty((rows * 64 * 2,), dtype=torch.int32, device=logits.device)      # 64 (value, index) pairs a row
    _call("ri_argmax", _dev(ids, "ids"), _dev(logits, "logits", torch.float32), _dev(ws, "workspace"), rows, vocab,
          _stream())
    return ids


# From this vocabulary size on a sampled row is cut over many workgroups (at 151,936 entries: 8 short
# launches instead of one long one).
SPLIT_SAMPLER_MIN_VOCAB = 16384


def sample(logits: torch.Tensor, uniform, temperature: float, top_k: int = 0, top_p: float = 1.0,
           penalty: float = 1.0, seen: torch.Tensor | None = None, seen_rows: torch.Tensor | None = None,
           split: bool | None = None) -> torch.Tensor:
    """int32 token per row of float32 ``logits``: repetition penalty over the ids marked in ``seen``
    (uint8 ``[*, vocab]``), greedy when the temperature is not positive, else temperature, top-k, top-p
    and one draw with ``uniform[r]`` in [0, 1).  ``split``: the many-workgroups form (the same token;
    by default for large vocabularies)."""
    rows, vocab = logits.shape
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    if split is None:
        split = vocab >= SPLIT_SAMPLER_MIN_VOCAB
    if split and temperature > 0:
        lib = load()
        lib.ri_sample_split_workspace_bytes.restype = ctypes.c_long
        lib.ri_sample_split_workspace_bytes.argtypes = [c_int]
        ws = torch.empty((lib.ri_sample_split_workspace_bytes(rows),), dtype=torch.uint8, device=logits.device)
        _call("ri_sample_split", _dev(out, "out"), _dev(logits, "logits", torch.float32),
              _opt(seen, "seen", torch.uint8), _opt(seen_rows, "seen_rows", torch.int32, (rows,)),
              _dev(uniform, "uniform", torch.float32, (rows,)), _dev(ws, "workspace"), rows, vocab, float(temperature),
              int(top_k), float(top_p), float(penalty), _stream())
        return out
    _call("ri_sample", _dev(out, "out"), _dev(logits, "logits", torch.float32),
          _opt(seen, "seen", torch.uint8), _opt(seen_rows, "seen_rows", torch.int32, (rows,)),
          _opt(uniform, "uniform", torch.float32, (rows,)), rows, vocab, float(temperature), int(top_k), float(top_p),
          float(penalty), _stream())
    return out


def mark_seen(seen: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor) -> None:
    """``seen[rows[i], tokens[i]] = 1``."""
    n = rows.shape[0]
    _call("ri_mark_seen", _dev(seen, "seen", torch.uint8), _dev(rows, "rows", torch.int32, (n,)),
          _dev(tokens, "tokens", torch.int32, (n,)), n, seen.shape[1], _stream())


# ---------------------------------------------------------------- attention
def qk_norm_rope_kv_write(qkv, q_gain, k_gain, eps, inv_freq, tok_pos, tok_seq, page_table, k_pages, v_pages,
                          heads: int, kv_heads: int, head_dim: int, cu_seqlens=None, max_new: int = 0) -> None:
    """In place on ``qkv: [T, (H + 2 Hkv) dh]``: per-head norm and rotation of q and k; k and v go to their
    pages.  ``inv_freq`` (float32 ``[r]``, ``r <= dh / 2``) rotates the first ``2 r`` elements of every head in
    pairs ``(i, i + r)``; what lies behind them is normed only.  With ``cu_seqlens`` (int32 ``[seqs + 1]``) and
    ``max_new`` values are written a page at a time."""
    tokens = qkv.shape[0]
    width = (heads + 2 * kv_heads) * head_dim
    if k_pages is None:                       # nothing goes to the cache: k is changed in place like q
        if v_pages is not None:
            raise ShapeError("key pages and value pages come together or not at all")
        num_pages, page_size = 0, 0
    else:
        num_pages, hkv, page_size, dh = k_pages.shape
        if (hkv, dh) != (kv_heads, head_dim) or tuple(v_pages.shape) != (num_pages, hkv, dh, page_size):
            raise ShapeError(f"pages are {list(k_pages.shape)} / {list(v_pages.shape)}, the mixer has {kv_heads} kv "
                             f"heads of {head_dim}")
    rot_dim = head_dim if inv_freq is None else 2 * inv_freq.shape[0]
    if inv_freq is not None and (inv_freq.dim() != 1 or not 2 <= rot_dim <= head_dim):
        raise ShapeError(f"inv_freq is {list(inv_freq.shape)}: a head of {head_dim} takes 1 to {head_dim // 2} frequencies")
    _call("ri_qk_norm_rope_kv_write", _dev(qkv, "qkv", None, (tokens, width)), code(qkv.dtype),
          _opt(q_gain, "q_gain", torch.float32, (head_dim,)), _opt(k_gain, "k_gain", torch.float32, (head_dim,)),
          float(eps), _opt(inv_freq, "inv_freq", torch.float32), rot_dim,
          _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _opt(cu_seqlens, "cu_seqlens", torch.int32), 0 if cu_seqlens is None else cu_seqlens.shape[0] - 1,
          int(max_new), _dev(page_table, "page_table", torch.int32), page_table.shape[1],
          _opt(k_pages, "k_pages"), _opt(v_pages, "v_pages"), code(qkv.dtype if k_pages is None else k_pages.dtype),
          tokens, heads, kv_heads, head_dim, page_size, num_pages, _stream())


def attention(qkv, k_pages, v_pages, tok_pos, tok_seq, page_table, heads: int, kv_heads: int, head_dim: int,
              window: int | None, scale: float) -> torch.Tensor:
    """Attention of every new token over its sequence's pages; q is the first ``H dh`` columns of ``qkv``."""
    tokens, stride = qkv.shape
    out = torch.empty((tokens, heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    _call("ri_attention", _dev(out, "out"), _dev(qkv, "qkv"), code(qkv.dtype), stride, _dev(k_pages, "k_pages"),
          _dev(v_pages, "v_pages"), code(k_pages.dtype), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(tok_seq, "tok_seq", torch.int32, (tokens,)), _dev(page_table, "page_table", torch.int32),
          page_table.shape[1], tokens, heads, kv_heads, head_dim, k_pages.shape[2], int(window or 0), float(scale),
          _stream())
    return out


MFMA_HEAD_DIMS = (32, 64, 128)
MAX_HEAD_DIM = 512          # what the general attention and q/k kernels take (any size from 1 up to it)


def mfma_attention_fits(dtype, head_dim: int, group: int, page_size: int, decode: bool) -> bool:
    """Whether the matrix-core attention kernels take this case (else the generic kernel does)."""
    return (dtype == torch.bfloat16 and head_dim in MFMA_HEAD_DIMS and page_size == 32
            and group <= (16 if decode else (64 if head_dim <= 64 else 32)))


def attention_prefill_bf16(qkv, k_pages, v_pages, cu_seqlens, tok_pos, page_table, seqs: int, max_new: int,
                           heads: int, kv_heads: int, head_dim: int, window: int | None, scale: float) -> torch.Tensor:
    """Matrix-core attention for any number of new tokens per sequence (bfloat16, pages of 32)."""
    tokens, stride = qkv.shape
    out = torch.empty((tokens, heads * head_dim), dtype=torch.bfloat16, device=qkv.device)
    _call("ri_attention_prefill_bf16", _dev(out, "out"), _dev(qkv, "qkv", torch.bfloat16), stride,
          _dev(k_pages, "k_pages", torch.bfloat16), _dev(v_pages, "v_pages", torch.bfloat16),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], seqs, max_new, heads, kv_heads, head_dim,
          k_pages.shape[2], int(window or 0), float(scale), _stream())
    return out


def decode_attention_runs(seqs: int, kv_heads: int, max_len: int) -> int:
    """The runs per sequence in which the decode attention's streaming kernel walks a step of this size, or 0
    where it takes one workgroup per chunk of 256 keys instead (host code only: it needs no GPU)."""
    chunks = _get("ri_attention_decode_chunks")(int(max_len))
    return _get("ri_attention_decode_streams")(int(seqs), int(kv_heads), chunks)


def decode_attention_streams(seqs: int, kv_heads: int, max_len: int) -> bool:
    """Whether ``attention_decode_bf16`` walks a step of this size with its streaming kernel (whole runs of a
    sequence's pages per workgroup) rather than with one workgroup per chunk of 256 keys."""
    return decode_attention_runs(seqs, kv_heads, max_len) > 0


def attention_decode_bf16(qkv, k_pages, v_pages, cu_seqlens, tok_pos, page_table, seqs: int, max_len: int,
                          heads: int, kv_heads: int, head_dim: int, window: int | None, scale: float,
                          tiled_out: bool = False):
    """Matrix-core attention for one new token per sequence; ``max_len`` bounds every sequence's length
    after this step (it sizes the grid and the workspace, not the result).  ``tiled_out``: the result as
    ``TiledRows`` (at most 64 sequences)."""
    tokens, stride = qkv.shape
    if tokens != seqs:
        raise ShapeError(f"decode attention takes one token per sequence, got {tokens} tokens for {seqs} sequences")
    chunks = _get("ri_attention_decode_chunks")(int(max_len))      # the kernels' own chunk size
    out = (TiledRows.empty(tokens, heads * head_dim, qkv.device) if tiled_out else
           torch.empty((tokens, heads * head_dim), dtype=torch.bfloat16, device=qkv.device))
    pieces = _get("ri_attention_decode_pieces")(int(seqs), int(kv_heads), int(heads), chunks)
    ws = torch.empty((seqs, heads, chunks * pieces, head_dim + 2), dtype=torch.float32, device=qkv.device)
    _call("ri_attention_decode_bf16", _dev(out.data if tiled_out else out, "out"), _dev(ws, "workspace"), _dev(qkv, "qkv", torch.bfloat16), stride,
          _dev(k_pages, "k_pages", torch.bfloat16), _dev(v_pages, "v_pages", torch.bfloat16),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], seqs, chunks, heads, kv_heads, head_dim,
          k_pages.shape[2], int(window or 0), float(scale), int(tiled_out), _stream())
    return out


def attention_decode_fused_bf16(qkv, q_gain, k_gain, eps, inv_freq, k_pages, v_pages, tok_pos, page_table, seqs: int,
                                max_len: int, heads: int, kv_heads: int, head_dim: int, window: int | None,
                                scale: float, tiled_out: bool = False):
    """A layer's decode attention from the raw ``qkv: [seqs, (H + 2 Hkv) dh]``: q/k norm, rotation, the new
    token's k and v into their pages and attention in one kernel, then the join.  ``tiled_out``: the result
    as ``TiledRows``."""
    tokens, stride = qkv.shape
    if tokens != seqs:
        raise ShapeError(f"decode attention takes one token per sequence, got {tokens} tokens for {seqs} sequences")
    num_pages, hkv, page_size, dh = k_pages.shape
    if (hkv, dh) != (kv_heads, head_dim) or tuple(v_pages.shape) != (num_pages, hkv, dh, page_size):
        raise ShapeError(f"pages are {list(k_pages.shape)} / {list(v_pages.shape)}, the mixer has {kv_heads} kv heads "
                         f"of {head_dim}")
    chunks = _get("ri_attention_decode_chunks")(int(max_len))      # the kernels' own chunk size
    out = (TiledRows.empty(tokens, heads * head_dim, qkv.device) if tiled_out else
           torch.empty((tokens, heads * head_dim), dtype=torch.bfloat16, device=qkv.device))
    pieces = _get("ri_attention_decode_pieces")(int(seqs), int(kv_heads), int(heads), chunks)
    ws = torch.empty((seqs, heads, chunks * pieces, head_dim + 2), dtype=torch.float32, device=qkv.device)
    half = head_dim // 2
    _call("ri_attention_decode_fused_bf16", _dev(out.data if tiled_out else out, "out"), _dev(ws, "workspace"),
          _dev(qkv, "qkv", torch.bfloat16), stride, _opt(q_gain, "q_gain", torch.float32, (head_dim,)),
          _opt(k_gain, "k_gain", torch.float32, (head_dim,)), float(eps),
          _opt(inv_freq, "inv_freq", torch.float32, (half,)), _dev(k_pages, "k_pages", torch.bfloat16),
          _dev(v_pages, "v_pages", torch.bfloat16), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], seqs, chunks, heads, kv_heads, head_dim,
          page_size, int(window or 0), float(scale), int(tiled_out), _stream())
    return out


# ---------------------------------------------------------------- products
def gemm_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x @ w.T`` in true 32-bit arithmetic; ``x`` float32 ``[M, K]``, ``w`` float32 or bfloat16 ``[N, K]``."""
    m, k = x.shape
    n = w.shape[0]
    out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _call("ri_gemm_f32", _dev(out, "out"), _dev(x, "x", torch.float32), _dev(w, "w", None, (n, k)), code(w.dtype),
          m, n, k, _stream())
    return out


def gemv_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype=torch.bfloat16, swiglu: bool = False) -> torch.Tensor:
    """``x @ w.T`` for up to 8 bfloat16 rows; with ``swiglu`` ``w`` is gate rows then up rows and the
    result is ``silu(gate) * up``."""
    m, k = x.shape
    n = w.shape[0] // 2 if swiglu else w.shape[0]
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _call("ri_gemv_bf16", _dev(out, "out"), code(out_dtype), _dev(x, "x", torch.bfloat16),
          _dev(w, "w", torch.bfloat16, (w.shape[0], k)), m, n, k, int(swiglu), _stream())
    return out


def pack_for_mfma(w: torch.Tensor, swiglu: bool = False) -> torch.Tensor:
    """A bfloat16 weight ``[N, K]`` cut into MFMA A-operand tiles: ``[ceil(N/16), ceil(K/32), 64, 8]``, lane
    ``l`` of a tile holding row ``l % 16`` and ``k = 8 * (l // 16) ..+8``, zero beyond N and K.  With
    ``swiglu`` the gate half and the up half of ``[2 N, K]`` are packed one after the other."""
    if swiglu:
        half = w.shape[0] // 2
        return torch.cat([pack_for_mfma(w[:half]), pack_for_mfma(w[half:])], 0)
    n, k = w.shape
    n16, k32 = -(-n // 16) * 16, -(-k // 32) * 32
    if (n16, k32) != (n, k):
        padded = torch.zeros((n16, k32), dtype=w.dtype, device=w.device)
        padded[:n, :k] = w
        w = padded
    tiles = w.view(n16 // 16, 16, k32 // 32, 4, 8).permute(0, 2, 3, 1, 4)      # [row tile, k tile, k group, row, 8]
    return tiles.reshape(n16 // 16, k32 // 32, 64, 8).contiguous()


TILED_X, TILED_OUT = 1, 2


class TiledRows:
    """Up to 64 bfloat16 rows of ``k`` columns in the order the matrix cores take them as an operand:
    ``data[ceil(m / 16), ceil(k / 32), 64, 8]``, lane ``l`` of a tile holding row ``l % 16`` of its 16 rows and
    the columns ``8 * (l // 16) ..+8`` of its 32.  A packed product, a norm or the decode attention writes its
    result this way for the packed product after it, which then loads a tile as one kilobyte in a row; rows
    beyond ``m`` and columns beyond ``k`` are never read."""

    def __init__(self, data: torch.Tensor, m: int, k: int):
        self.data, self.shape = data, (m, k)
        self.dtype, self.device = data.dtype, data.device

    @staticmethod
    def empty(m: int, k: int, device) -> "TiledRows":
        if not 1 <= m <= 64:
            raise ShapeError(f"tiled rows hold 1 to 64 rows, not {m}")
        return TiledRows(torch.empty((-(-m // 16), -(-k // 32), 64, 8), dtype=torch.bfloat16, device=device), m, k)

    def rows(self) -> torch.Tensor:
        """The same values row-major, ``[m, k]``."""
        m, k = self.shape
        row_tiles, tiles = self.data.shape[:2]
        return (self.data.view(row_tiles, tiles, 4, 16, 8).permute(0, 3, 1, 2, 4)
                .reshape(row_tiles * 16, tiles * 32)[:m, :k].contiguous())


def as_rows(x):
    """A tensor for code that wants plain rows."""
    return x.rows() if isinstance(x, TiledRows) else x


def gemm_skinny_packed_bf16(x, wpacked: torch.Tensor, n: int, out_dtype=torch.bfloat16,
                            swiglu: bool = False, parts: int = 1, tiled_out: bool = False):
    """``x @ w.T`` for up to 16 bfloat16 rows (a tensor or ``TiledRows``) with ``w`` packed by
    ``pack_for_mfma``; ``n`` is the number of output columns (rows of w; of its gate half with ``swiglu``).
    With ``parts > 1`` K is cut into that many pieces and the result is their float32 sums ``[parts, M, n]``,
    for a consumer that adds them.  With ``tiled_out`` the bfloat16 result comes as ``TiledRows``."""
    m, k = x.shape
    row_tiles = -(-n // 16)
    want = (row_tiles * (2 if swiglu else 1), -(-k // 32), 64, 8)
    if tuple(wpacked.shape) != want:
        raise ShapeError(f"packed weight is {list(wpacked.shape)}, a product with n {n}, k {k} wants {list(want)}")
    if tiled_out and (parts != 1 or out_dtype != torch.bfloat16):
        raise ShapeError("a tiled result is bfloat16 and whole")
    flags = (TILED_X if isinstance(x, TiledRows) else 0) | (TILED_OUT if tiled_out else 0)
    xd = _dev(x.data, "x", torch.bfloat16) if isinstance(x, TiledRows) else _dev(x, "x", torch.bfloat16)
    if tiled_out:
        out = TiledRows.empty(m, n, x.device)
        od = _dev(out.data, "out")
    else:
        out = torch.empty((m, n) if parts == 1 else (parts, m, n), dtype=out_dtype, device=x.device)
        od = _dev(out, "out")
    _call("ri_gemm_skinny_packed_bf16", od, code(out_dtype), xd, _dev(wpacked, "wpacked", torch.bfloat16), m, n, k,
          int(swiglu), int(parts), flags, _stream())
    return out


class NormedLater:
    """Rows of a residual stream whose RMSNorm is left to the product that reads them:
    ``xg = bfloat16(r * gain)`` and partial sums of ``r^2`` per row, ``[M, partials]``; the
    normed rows are ``xg / sqrt(ssq.sum(1) / dim + eps)``.  ``xg`` is a tensor or ``TiledRows``."""

    def __init__(self, xg, ssq: torch.Tensor, eps: float, dim: int):
        self.xg, self.ssq, self.eps, self.dim = xg, ssq, float(eps), int(dim)
        self.shape, self.dtype, self.device = xg.shape, xg.dtype, xg.device


def finish_norm(later: NormedLater) -> torch.Tensor:
    """The normed bfloat16 rows ``[M, dim]`` of a ``NormedLater``, for a reader that cannot take the norm
    over (``xg`` was rounded once already, so this differs from the plain norm by one more rounding)."""
    xg = later.xg
    tiled = isinstance(xg, TiledRows)
    m, dim = xg.shape
    out = torch.empty((m, dim), dtype=torch.bfloat16, device=later.device)
    _call("ri_finish_norm", _dev(out, "out"), _dev(xg.data if tiled else xg, "xg", torch.bfloat16),
          _dev(later.ssq, "ssq", torch.float32, (m, later.ssq.shape[1])), later.ssq.shape[1], later.eps, later.dim, m,
          int(tiled), _stream())
    return out


def gemm_mid_packed_bf16(x, wpacked: torch.Tensor, n: int, out_dtype=torch.bfloat16, swiglu: bool = False,
                         tiled_out: bool = False):
    """``x @ w.T`` for up to 64 bfloat16 rows (a tensor or ``TiledRows``) with ``w`` packed by
    ``pack_for_mfma``: the packed product for the steps of 17 to 64 tokens.  ``tiled_out``: the bfloat16
    result as ``TiledRows``."""
    m, k = x.shape
    row_tiles = -(-n // 16)
    want = (row_tiles * (2 if swiglu else 1), -(-k // 32), 64, 8)
    if tuple(wpacked.shape) != want:
        raise ShapeError(f"packed weight is {list(wpacked.shape)}, a product with n {n}, k {k} wants {list(want)}")
    if tiled_out and out_dtype != torch.bfloat16:
        raise ShapeError("a tiled result is bfloat16")
    x_tiled = isinstance(x, TiledRows)
    out = TiledRows.empty(m, n, x.device) if tiled_out else torch.empty((m, n), dtype=out_dtype, device=x.device)
    _call("ri_gemm_mid_packed_bf16", _dev(out.data if tiled_out else out, "out"), code(out_dtype),
          _dev(x.data if x_tiled else x, "x", torch.bfloat16), _dev(wpacked, "wpacked", torch.bfloat16), m, n, k,
          int(swiglu), (TILED_X if x_tiled else 0) | (TILED_OUT if tiled_out else 0), _stream())
    return out


def compute_units() -> int:
    """Compute units of the current device (256 where there is none): what the rules that size launches
    count workgroups against."""
    return int(_get("ri_compute_units")())


def wide_product_plan(n: int, k: int, swiglu: bool = False, rows: int = 64) -> tuple[int, int]:
    """``(waves, parts)``: how many wavefronts a workgroup of ``gemm_wide_packed_bf16`` should have and into how
    many stretches of K it should cut a product of ``rows`` rows with an ``n x k`` matrix (host code only): with the
    activation K whole and the wavefronts that fill the compute units more evenly; without it, from 17 rows on,
    what makes a compute unit fetch the fewest bytes."""
    waves, parts = ctypes.c_int(0), ctypes.c_int(0)
    if swiglu:
        if rows > 64:
            raise ShapeError("more than 64 rows go without the activation")
        _call("ri_gemm_wide_packed_bf16_plan", int(n), int(k), 1, ctypes.addressof(waves), ctypes.addressof(parts))
    else:
        _call("ri_gemm_wide_stretch_plan", int(rows), int(n), int(k), ctypes.addressof(waves), ctypes.addressof(parts))
    return waves.value, parts.value


def gemm_wide_packed_bf16(x, wpacked: torch.Tensor, n: int, out_dtype=torch.bfloat16, swiglu: bool = False,
                          parts: int = 1, tiled_out: bool = False, depth: int = 2, waves: int = 4):
    """``x @ w.T`` for up to 64 bfloat16 rows (a tensor or ``TiledRows``) with ``w`` packed by ``pack_for_mfma``,
    the tiles of x shared by a workgroup's wavefronts through LDS: the product for steps of 17 to 64 tokens.
    65 to 256 plain rows (past 128 in two passes over the weights): float32 sums in rows (``waves`` and ``parts``
    from ``wide_product_plan(..., rows=m)``), ``depth`` 1; with ``swiglu`` 65 to 128 plain rows where the plan says
    five to eight wavefronts, K whole.
    ``parts > 1``: K in that many stretches, the result their float32 sums ``[parts, M, n]`` for a reader
    that adds them (with ``swiglu`` ``[parts, M, 2 n]``, gate sums then up sums, the activation left to
    ``sum_parts``).  ``tiled_out``: the bfloat16 result as ``TiledRows``.  ``waves``: wavefronts (row tiles) a
    workgroup, 3 or 4, with the activation at ``depth`` 1 up to 8 (``wide_product_plan``); the sums do not depend on it."""
    m, k = x.shape
    row_tiles = -(-n // 16)
    want = (row_tiles * (2 if swiglu else 1), -(-k // 32), 64, 8)
    if tuple(wpacked.shape) != want:
        raise ShapeError(f"packed weight is {list(wpacked.shape)}, a product with n {n}, k {k} wants {list(want)}")
    if m > 64:
        if tiled_out or isinstance(x, TiledRows) or (not swiglu and out_dtype != torch.float32) or (swiglu and (parts != 1 or m > 128)):
            raise ShapeError("more than 64 rows: plain rows in and out; float32 sums without the activation, "
                             "or up to 128 rows with it and K whole")
        depth = 1
    if parts != 1 and (out_dtype != torch.float32 or tiled_out):
        raise ShapeError("a product in parts has float32 sums in rows")
    if tiled_out and out_dtype != torch.bfloat16:
        raise ShapeError("a tiled result is bfloat16")
    x_tiled = isinstance(x, TiledRows)
    if tiled_out:
        out = TiledRows.empty(m, n, x.device)
    else:
        out = torch.empty((m, n) if parts == 1 else (parts, m, 2 * n if swiglu else n), dtype=out_dtype, device=x.device)
    _call("ri_gemm_wide_packed_bf16", _dev(out.data if tiled_out else out, "out"), code(out_dtype),
          _dev(x.data if x_tiled else x, "x", torch.bfloat16), _dev(wpacked, "wpacked", torch.bfloat16), m, n, k,
          int(swiglu), int(parts), (TILED_X if x_tiled else 0) | (TILED_OUT if tiled_out else 0), int(depth),
          int(waves), _stream())
    return out


def sum_parts(parts: torch.Tensor, out_dtype=torch.bfloat16, tiled_out: bool = False, swiglu: bool = False):
    """``parts.sum(0)`` of float32 ``[parts, M, n]``, added in order, as ``out_dtype`` (bfloat16 also as
    ``TiledRows``); with ``swiglu`` the rows are gate sums then up sums and the result ``silu(gate) * up``."""
    p, m, n = parts.shape
    if swiglu:
        if n % 2:
            raise ShapeError(f"gate and up sums side by side have an even width, not {n}")
        n //= 2
    out = TiledRows.empty(m, n, parts.device) if tiled_out else torch.empty((m, n), dtype=out_dtype, device=parts.device)
    _call("ri_sum_parts", _dev(out.data if tiled_out else out, "out"), code(torch.bfloat16 if tiled_out else out_dtype),
          _dev(parts, "parts", torch.float32), p, m, n, int(swiglu), int(tiled_out), _stream())
    return out


def linked_product(x, w: torch.Tensor, n: int, packed: bool, out_dtype=torch.bfloat16, swiglu: bool = False,
                   residual: torch.Tensor | None = None, next_gain: torch.Tensor | None = None,
                   next_eps: float = 0.0, tiled_out: bool = False):
    """A decode-size product that does the RMSNorm before it, the residual add and the RMSNorm's
    preparation after it, or both, in the same kernel.

    ``x`` is bfloat16 rows (a tensor or ``TiledRows``) or a ``NormedLater``; ``w`` the row-major weight
    (``packed`` false: up to 8 rows, one wavefront per weight row) or its MFMA tiles (``packed`` true: up to
    16 rows).  With ``residual`` (float32 ``[M, n]``, updated in place to ``residual + x @ w.T``) the result
    is the ``NormedLater`` of the new residual for a norm with ``next_gain`` and ``next_eps``; else the
    product.  ``tiled_out`` (packed only) asks for the bfloat16 rows of the result as ``TiledRows``."""
    later = x if isinstance(x, NormedLater) else None
    xr = later.xg if later else x
    if not packed:
        xr, tiled_out = as_rows(xr), False
    m, k = xr.shape
    name = "ri_gemm_skinny_packed_bf16" if packed else "ri_gemv_bf16"
    if packed:
        want = (-(-n // 16) * (2 if swiglu else 1), -(-k // 32), 64, 8)
        if tuple(w.shape) != want:
            raise ShapeError(f"packed weight is {list(w.shape)}, a product with n {n}, k {k} wants {list(want)}")
        wd = _dev(w, "wpacked", torch.bfloat16)
    else:
        wd = _dev(w, "w", torch.bfloat16, (n * (2 if swiglu else 1), k))
    x_tiled = isinstance(xr, TiledRows)
    xd = _dev(xr.data, "x", torch.bfloat16) if x_tiled else _dev(xr, "x", torch.bfloat16, (m, k))
    # the packed kernel takes the layouts of x and of its result as one more argument
    layout = ((TILED_X if x_tiled else 0) | (TILED_OUT if tiled_out else 0),) if packed else ()
    if later is not None:
        ssq_in = _dev(later.ssq, "ssq", torch.float32, (m, later.ssq.shape[1]))
        n_in, eps, dim = later.ssq.shape[1], later.eps, later.dim
        if dim != k:
            raise ShapeError(f"rows normed over {dim} elements into a product over {k}")
    else:
        ssq_in, n_in, eps, dim = None, 0, 0.0, 0
    if residual is None:
        if tiled_out and out_dtype != torch.bfloat16:
            raise ShapeError("a tiled result is bfloat16")
        out = TiledRows.empty(m, n, xr.device) if tiled_out else torch.empty((m, n), dtype=out_dtype, device=xr.device)
        _call(name + "_linked", _dev(out.data if tiled_out else out, "out"), code(out_dtype), xd, wd, m, n, k,
              int(swiglu), ssq_in, n_in, eps, dim, None, None, None, None, *layout, _stream())
        return out
    if swiglu:
        raise ShapeError("a gate|up product does not feed the residual stream")
    partials = _get("ri_gemm_skinny_packed_bf16_partials")(n) if packed else _get("ri_gemv_bf16_partials")(n, k)
    xg = TiledRows.empty(m, n, xr.device) if tiled_out else torch.empty((m, n), dtype=torch.bfloat16, device=xr.device)
    ssq = torch.empty((m, partials), dtype=torch.float32, device=xr.device)
    _call(name + "_linked", None, code(torch.bfloat16), xd, wd, m, n, k, 0,
          ssq_in, n_in, eps, dim, _dev(residual, "residual", torch.float32, (m, n)),
          _dev(next_gain, "next_gain", torch.float32, (n,)), _dev(xg.data if tiled_out else xg, "xg"), _dev(ssq, "ssq"),
          *layout, _stream())
    return NormedLater(xg, ssq, next_eps, n)
