"""What parts need from their surroundings at run time: the device, the compute
dtype, and the matrix product that fits both."""
from __future__ import annotations

import functools

import torch

from ..errors import KernelError, ShapeError
from ..kernels import ops


@functools.lru_cache(maxsize=None)
def _wide_plan(n: int, k: int, swiglu: bool, rows: int = 64) -> tuple[int, int]:
    """``ops.wide_product_plan``, asked once per matrix size and tile of 16 rows."""
    return ops.wide_product_plan(n, k, swiglu, rows)

# Which product kernel runs, by the number of rows of x (bfloat16; the measurements behind every constant
# here are written up with the design notes, under "Which product kernel serves which step"):
#   1 row      one wavefront per weight row (ops.gemv_bf16).
#   2-16 rows  the matrix-core kernel on weights packed into MFMA tiles ahead of time, where a part asked for the
#              packed copy (the rule is _packed_pays below); it hands its rows to the next packed product in the
#              operand's order (ops.TiledRows) and does the norms around it.
#   17-64      the wide kernel (tiles of x shared through LDS) where the reader adds stretches of K or the
#              gate|up pairs fill the machine; the packed kernel with two or four tiles of x on small matrices
#              and up to 32 rows of tiled x; else the library.
#   65-128     the wide kernel with two row tiles a wavefront for matrices of long rows whose reader adds stretches
#              of K (`down`; up to 256 rows for the longest), and for the largest gate|up pairs; else the library.
#   more       the vendor library (the reference hands every product to one: src/cuda/mod.rs:186-232).
GEMV_MAX_ROWS = 1
SKINNY_MAX_ROWS = 16
MID_MAX_ROWS = 64
MID_MAX_BYTES = 20_000_000       # up to this size the packed kernel beats the library at 17 to 64 plain rows
MID_TILED_ROWS = 32              # and up to this many rows when the rows come tiled,
MID_TILED_BYTES = 64_000_000     # on matrices up to this size (7168 x 5120 draws level with the library, 10240 x 5120 loses: 28 us to 20)
WIDE_MIN_K = 4096                # rows shorter than this leave the wide kernel's stretches too little to do
WIDE_MIN_ROWS = 17
PAIRS_MAX_ROWS = 128             # 65 to 128 rows: the wide kernel with two row tiles a wavefront, where the library does badly:
PAIRS_MIN_K = 8192               # matrices of long rows (and at least twice as long as there are rows: `down`)
PAIRS_MORE_ROWS = 256            # and in two passes up to this many rows where the rows have PACKED_LONG_K elements and more
SMALL_ONLY_ROWS = 64             # a matrix packed for small steps alone stays on the wide kernel up to this many rows
# (5,120 x 8,192 at 32 / 48 / 64 rows: 20 / 24 / 29 us against the library's 19 to 34 / 30 / 23; 5,120 x 5,120: 15 / 18 / 21 against 19 / 20 / 19;
# with three stretches of 80 groups of four wavefronts 24 and 18 us at 64 rows: a step of 49 to 64 sequences 1 to 1.6% shorter at those sizes)
WIDE_GATED_FILL = 0.75            # gate|up goes to the wide kernel where its workgroups fill this share of the rounds,
WIDE_GATED_ROWS = 48             # and up to this many rows whatever they fill, if the packed kernel of 17 to 64 rows is no match:
WIDE_GATED_BYTES = 64_000_000    # pairs larger than this (smaller ones, up to 32 tiled rows, are that kernel's)
SPLIT_K = 4096                   # pieces of a long K (PACKED_LONG_K and more) whose sums the next norm adds
# Which matrices get a packed copy for 2 to 16 rows (the gate|up matrix always does: its activation rides in
# the kernel): up to 40 MB always; up to PACKED_MAX_BYTES unless the last round of workgroups (one per 16 rows)
# would leave most compute units idle; rows of PACKED_LONG_K elements and more always, cut into parts.
PACKED_MAX_BYTES = 101_000_000
PACKED_LONG_K = 16384


@functools.lru_cache(maxsize=None)
def _compute_units() -> int:
    return ops.compute_units()


def _packed_pays(n: int, k: int) -> bool:
    if k >= PACKED_LONG_K or n * k * 2 <= 40_000_000:
        return True
    tiles = -(-n // 16)
    cus = _compute_units()
    last_round = tiles % cus
    return n * k * 2 <= PACKED_MAX_BYTES and not (tiles > cus and 0 < last_round < cus // 2)


class PackedWeight:
    """A bfloat16 weight as the library product wants it (row-major) and, for decode-size products,
    packed into MFMA tiles."""

    def __init__(self, w: torch.Tensor, packed: torch.Tensor | None, swiglu: bool):
        self.w, self.packed, self.swiglu = w, packed, swiglu
        self.n = w.shape[0] // 2 if swiglu else w.shape[0]
        self.k = w.shape[1]
        # a long K is cut into pieces of 4096 whose float32 sums the next norm adds up: more workgroups
        # stream the weights (768 instead of 256 for 4096 x 12288), and the sum is never rounded to 16 bits
        self.parts = self.k // SPLIT_K if (not swiglu and self.k >= PACKED_LONG_K) else 1
        # 2 to 16 rows into the residual stream go to the wide kernel (set by Runtime.pack: see there)
        self.small_wide = False
        self.small_only = False      # the packed copy was made for that alone: larger steps stay where they were


class Runtime:
    """``dtype`` is the compute dtype: bfloat16 (16-bit activations and cache,
    float32 statistics and residual stream) or float32 (everything in true 32-bit;
    weights stay as stored and are widened exactly inside the kernels).

    ``invariant`` (bfloat16 only; float32 is so by itself): every step runs the same form of every kernel whatever
    its size, so that a request's logits are the same bits alone and in any batch, whole and token by token, as a
    graph and launched from the host.  The bfloat16 path otherwise chooses the product kernel by the number of rows,
    the attention kernel by the number of sequences and leaves small steps' norms to the products, and each form
    rounds at other places.  Here every product is the packed kernel for 17 to 64 rows in slices of 64 rows
    (a row's sums in it do not depend on the other rows), every norm the plain kernel, the q/k norm, rotation
    and cache write the kernel of one wavefront per token and head, and the attention the prompt kernel for
    single tokens too (a token's sums run over its sequence's pages in order whatever shares its tile), or the
    generic kernel, whose key tiles start at fixed positions, where that one does not take the sizes.  It is
    several times slower on prompts; it is for runs that must reproduce bit for bit."""

    def __init__(self, device="cuda:0", dtype=torch.bfloat16, invariant: bool = False):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ShapeError(f"compute dtype {dtype} is neither bfloat16 nor float32")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"this library computes on the GPU only, not on {self.device}")
        self.dtype = dtype
        self.invariant = bool(invariant) and dtype == torch.bfloat16
        self._mm_out_dtype = None

    # ---- weights
    def place_matrix(self, w: torch.Tensor) -> torch.Tensor:
        """A linear or embedding weight on the device: bfloat16 for bfloat16 compute,
        as stored for float32 compute."""
        w = w.to(self.device, non_blocking=False)
        if self.dtype == torch.bfloat16 and w.dtype != torch.bfloat16:
            w = w.to(torch.bfloat16)
        return w.contiguous()

    def place_gain(self, g: torch.Tensor) -> torch.Tensor:
        """Norm gains are used in float32 whatever they are stored in
        (the reference: src/models/qwen3.rs:184, src/models/cuda.rs:45)."""
        return g.to(self.device).to(torch.float32).contiguous()

    # ---- products
    def linear(self, x: torch.Tensor, w: torch.Tensor, out_dtype=None) -> torch.Tensor:
        """``x @ w.T`` with float32 accumulation; no bias anywhere in this family
        (the reference: src/ops/linear.rs:7-19)."""
        out_dtype = out_dtype or self.dtype
        if x.shape[1] != w.shape[1]:
            raise ShapeError(f"linear: x has {x.shape[1]} columns, the weight {w.shape[1]}")
        if self.dtype == torch.float32:
            return ops.gemm_f32(x, w)
        m, k = x.shape
        if m <= GEMV_MAX_ROWS and k % 8 == 0:
            if isinstance(x, ops.NormedLater):
                return ops.linked_product(x, w, w.shape[0], False, out_dtype)
            return ops.gemv_bf16(ops.as_rows(x), w, out_dtype)
        return self._library_mm(self.normed_now(x), w, out_dtype)

    @staticmethod
    def normed_now(x):
        """The rows of a ``NormedLater`` for a product that cannot do the norm itself."""
        if not isinstance(x, ops.NormedLater):
            return ops.as_rows(x)
        return ops.finish_norm(x)

    def pack(self, w: torch.Tensor, swiglu: bool = False, always: bool = False, parts_ok: bool = False) -> PackedWeight:
        """A placed weight, with a packed copy where the packed kernel is the faster one for 2 to 16
        rows (bfloat16 compute only), or wherever it can be used when the caller says ``always``.
        ``parts_ok``: the product's reader adds stretches of K (the residual stream's next norm).  Then a matrix
        that the packed kernel serves badly at 2 to 16 rows, one whose row tiles leave most compute units idle in
        their last round (5,120 rows) or whose long rows it cuts into parts itself (K of 16,384 and more), goes to
        the wide kernel there, which shares the rows of x through LDS and plans its stretches for the machine
        (5,120 x 5,120 at 8 rows: 11 us against the library's 19; 5,120 x 25,600: 41 against 51)."""
        n, k = w.shape
        if self.invariant and k % 8:
            raise ShapeError(f"the invariant mode's product takes rows of a multiple of 8 elements, not {k}")
        pays = always or swiglu or self.invariant or _packed_pays(n, k)
        small_wide = (parts_ok and not swiglu and not self.invariant and k >= WIDE_MIN_K
                      and (not pays or k >= PACKED_LONG_K))
        if self.dtype != torch.bfloat16 or k % 8 or not (pays or small_wide):
            return PackedWeight(w, None, swiglu)
        pw = PackedWeight(w, ops.pack_for_mfma(w, swiglu), swiglu)
        pw.small_wide, pw.small_only = small_wide, small_wide and not pays
        return pw

    @staticmethod
    def _mid_pays(pw: PackedWeight, m: int, tiled: bool) -> bool:
        """Whether the packed kernel for 17 to 64 rows beats the library's product (and, for gate|up, its
        activation kernel) on this matrix."""
        size = pw.w.shape[0] * pw.k * 2
        if size <= MID_MAX_BYTES:
            return True
        return tiled and m <= MID_TILED_ROWS and size <= MID_TILED_BYTES

    @staticmethod
    def _wide_gated(pw: PackedWeight, m: int) -> bool:
        """Whether the wide kernel takes a gate|up pair at 17 to 64 rows: up to WIDE_GATED_ROWS rows whenever the
        pair is too large for the packed kernel of those rows (which takes twice as long for twice the rows);
        beyond, where its workgroups (of three or four wavefronts, K whole) fill the compute units evenly; else a
        quarter of the machine idles and the library with its activation kernel is as fast."""
        if pw.packed is None:
            return False
        size = pw.w.shape[0] * pw.k * 2
        if m <= WIDE_GATED_ROWS and (size > WIDE_GATED_BYTES or (m > MID_TILED_ROWS and size > MID_MAX_BYTES)):
            return True
        waves, parts = _wide_plan(pw.n, pw.k, True)
        groups = -(-(-(-pw.n // 16)) // waves) * parts
        cus = _compute_units()
        return groups / (-(-groups // cus) * cus) >= WIDE_GATED_FILL

    def takes_tiled(self, pw: PackedWeight, m: int, parts_ok: bool = False) -> bool:
        """Whether the product of ``m`` rows with this weight (called with this ``parts_ok``) runs on a packed
        kernel: whoever makes its rows then makes them as ``ops.TiledRows``."""
        if self.dtype != torch.bfloat16 or pw.packed is None or pw.k % 8 or self.invariant:
            return False
        if pw.small_only:                                        # a packed copy made for small steps into the stream alone:
            return parts_ok and 2 < m <= SMALL_ONLY_ROWS         # the wide kernel takes those, nothing else of it
        if GEMV_MAX_ROWS < m <= SKINNY_MAX_ROWS:
            return True
        if WIDE_MIN_ROWS <= m <= MID_MAX_ROWS and (self._wide_gated(pw, m) if pw.swiglu
                                                   else parts_ok and pw.k >= WIDE_MIN_K):
            return True                                          # the wide kernel (where the reader adds its parts)
        return SKINNY_MAX_ROWS < m <= MID_MAX_ROWS and self._mid_pays(pw, m, True)

    def linear_packed(self, x, pw: PackedWeight, out_dtype=None, parts_ok: bool = False, link=None,
                      tiled_out: bool = False):
        """``x @ w.T`` (or ``silu(x @ gate.T) * (x @ up.T)`` for a fused gate|up weight) with the kernel
        that fits the number of rows.  With ``parts_ok`` the result may be ``[parts, M, N]`` float32, the
        sums over pieces of K, for a consumer that adds them (the residual stream's next norm).

        ``x`` may be a ``NormedLater`` or ``TiledRows``.  With ``tiled_out`` the caller takes the result as
        ``TiledRows`` where the packed kernel makes it (2 to 16 rows): the layout the next packed product
        reads fastest.  With ``link`` (the residual stream's offer to the last product of
        a branch) a kernel that can adds the result into the stream and prepares the next norm; the
        return value is then ``(NormedLater, norm)`` for the stream instead of a tensor."""
        out_dtype = out_dtype or self.dtype
        m = x.shape[0]
        if self.invariant:
            # one kernel for every step: a row's sums in it depend on the row and the matrix alone
            x = self.normed_now(x)
            outs = [ops.gemm_mid_packed_bf16(x[i:i + MID_MAX_ROWS], pw.packed, pw.n, out_dtype, swiglu=pw.swiglu)
                    for i in range(0, m, MID_MAX_ROWS)]
            return outs[0] if len(outs) == 1 else torch.cat(outs, 0)
        if self.dtype == torch.bfloat16 and pw.k % 8 == 0:
            later = isinstance(x, ops.NormedLater)
            mine = None
            if (max(GEMV_MAX_ROWS, 2 if pw.small_only else 0) < m <= SKINNY_MAX_ROWS and pw.small_wide and parts_ok):
                # (the parts beat a link to the next norm, as they do for the packed kernel's own; two rows of a
                # matrix that had no packed copy stay with the kernel of one wavefront a row, which takes the link)
                x = self.normed_now(x) if later else x
                waves, parts = _wide_plan(pw.n, pw.k, False, -(-m // 16) * 16)
                return ops.gemm_wide_packed_bf16(x, pw.packed, pw.n, torch.float32, parts=parts, depth=1, waves=waves)
            if (SKINNY_MAX_ROWS // 2 < m <= SKINNY_MAX_ROWS and pw.swiglu and pw.packed is not None and not later
                    and pw.k >= WIDE_MIN_K):
                # 9 to 16 rows of a gate|up pair whose input is plain rows (the norm before it was a kernel of its
                # own): the packed kernel loads every row of x once per 16 rows of weights there (its form that
                # serves two steps with one load takes 8 rows), the wide one shares them through LDS (16 rows at
                # Qwen3-8B, 14B and 32B sizes: 33, 64 and 86 us against 35, 67 and 95)
                waves, _ = _wide_plan(pw.n, pw.k, True)
                return ops.gemm_wide_packed_bf16(x, pw.packed, pw.n, out_dtype, swiglu=True, depth=1, waves=waves,
                                                 tiled_out=tiled_out and out_dtype == torch.bfloat16)
            if m <= GEMV_MAX_ROWS or (m <= 2 and (pw.packed is None or pw.small_only)):
                mine = (pw.w, False)
            elif m <= SKINNY_MAX_ROWS and pw.packed is not None and not pw.small_only:
                mine = (pw.packed, True)
            if mine is not None:
                in_parts = mine[1] and parts_ok and pw.parts > 1        # very long rows: parts beat the link
                tiles = mine[1] and tiled_out and out_dtype == torch.bfloat16
                if link is not None and not pw.swiglu and not in_parts and link.residual.shape == (m, pw.n):
                    made = ops.linked_product(x, mine[0], pw.n, mine[1], residual=link.residual,
                                              next_gain=link.gain, next_eps=link.eps,
                                              tiled_out=mine[1] and link.tiled)
                    return (made, link.norm)
                if in_parts:
                    x = self.normed_now(x) if later else x
                    return ops.gemm_skinny_packed_bf16(x, pw.packed, pw.n, torch.float32, parts=pw.parts)
                if later:
                    return ops.linked_product(x, mine[0], pw.n, mine[1], out_dtype, swiglu=pw.swiglu, tiled_out=tiles)
                if not mine[1]:
                    return ops.gemv_bf16(ops.as_rows(x), pw.w, out_dtype, swiglu=pw.swiglu)
                return ops.gemm_skinny_packed_bf16(x, pw.packed, pw.n, out_dtype, swiglu=pw.swiglu, tiled_out=tiles)
            if (WIDE_MIN_ROWS <= m <= MID_MAX_ROWS and pw.packed is not None and parts_ok and not pw.swiglu
                    and pw.k >= WIDE_MIN_K and not (pw.small_only and m > SMALL_ONLY_ROWS)):
                # 17 to 64 rows into the residual stream: K in stretches, every stretch a workgroup that shares the tiles of x
                # through LDS; the stream's next norm adds the stretches' sums
                x = self.normed_now(x) if later else x
                waves, parts = _wide_plan(pw.n, pw.k, False, -(-m // 16) * 16)
                return ops.gemm_wide_packed_bf16(x, pw.packed, pw.n, torch.float32, parts=parts, depth=1, waves=waves)
            if (MID_MAX_ROWS < m <= (PAIRS_MORE_ROWS if pw.k >= PACKED_LONG_K else PAIRS_MAX_ROWS) and pw.packed is not None
                    and parts_ok and not pw.swiglu and pw.k >= PAIRS_MIN_K and pw.k >= 2 * pw.n):
                # 65 to 128 rows against a matrix of long rows whose result goes into the residual stream (`down`):
                # the wide kernel with two row tiles a wavefront, K in stretches that the stream's next norm adds
                # (the longest rows up to 256 rows of x, in two passes over the weights)
                x = self.normed_now(x) if later else x
                x = x.rows() if isinstance(x, ops.TiledRows) else x
                waves, parts = _wide_plan(pw.n, pw.k, False, -(-m // 16) * 16)
                return ops.gemm_wide_packed_bf16(x, pw.packed, pw.n, torch.float32, parts=parts, depth=1, waves=waves)
            if MID_MAX_ROWS < m <= PAIRS_MAX_ROWS and pw.swiglu and pw.packed is not None:
                # 65 to 128 rows of the largest gate|up pairs (those that take five to eight wavefronts a workgroup)
                waves, _ = _wide_plan(pw.n, pw.k, True)
                if waves > 4:
                    x = self.normed_now(x) if later else x
                    x = x.rows() if isinstance(x, ops.TiledRows) else x
                    return ops.gemm_wide_packed_bf16(x, pw.packed, pw.n, out_dtype, swiglu=True, depth=1, waves=waves)
            if WIDE_MIN_ROWS <= m <= MID_MAX_ROWS and pw.swiglu and self._wide_gated(pw, m):
                x = self.normed_now(x) if later else x
                waves, _ = _wide_plan(pw.n, pw.k, True)
                return ops.gemm_wide_packed_bf16(x, pw.packed, pw.n, out_dtype, swiglu=True, depth=1, waves=waves,
                                                 tiled_out=tiled_out and out_dtype == torch.bfloat16)
            if (SKINNY_MAX_ROWS < m <= MID_MAX_ROWS and pw.packed is not None
                    and self._mid_pays(pw, m, isinstance(x, ops.TiledRows))):
                x = self.normed_now(x) if later else x
                return ops.gemm_mid_packed_bf16(x, pw.packed, pw.n, out_dtype, swiglu=pw.swiglu,
                                                tiled_out=tiled_out and out_dtype == torch.bfloat16)
        y = self.linear(x, pw.w, None if pw.swiglu else out_dtype)
        return ops.swiglu(y, tiled_out=tiled_out) if pw.swiglu else y

    def _library_mm(self, x, w, out_dtype):
        # The reference hands every product to a vendor library (src/cuda/mod.rs:186-232);
        # so does this path, for the shapes its own kernels do not cover.
        if out_dtype == torch.float32:
            if self._mm_out_dtype is None:
                try:
                    torch.mm(x[:1], w[:1].t(), out_dtype=torch.float32)
                    self._mm_out_dtype = True
                except (TypeError, RuntimeError):
                    self._mm_out_dtype = False
            if self._mm_out_dtype:
                return torch.mm(x, w.t(), out_dtype=torch.float32)
            return torch.mm(x, w.t()).to(torch.float32)
        return torch.mm(x, w.t())
