"""What parts need from their surroundings at run time: the device, the compute
dtype, and the matrix product that fits both."""
from __future__ import annotations

import torch

from ..errors import KernelError, ShapeError
from ..kernels import ops

# Which product kernel runs, by the number of rows of x (measured on MI355X at Qwen3-8B sizes with the
# weights streamed from HBM): the one-wavefront-per-row kernel is fastest for one or two rows
# (5.1 to 5.5 TB/s on the large matrices); from three rows on it is bound by its vector
# arithmetic and the vendor library's product is faster (4.2 to 4.9 TB/s); the matrix-core kernel of
# this library wins only on matrices up to 4096 x 4096.
GEMV_MAX_ROWS = 2
SKINNY_MAX_ROWS = 16
SKINNY_MAX_SIDE = 4096


class Runtime:
    """``dtype`` is the compute dtype: bfloat16 (16-bit activations and cache,
    float32 statistics and residual stream) or float32 (everything in true 32-bit;
    weights stay as stored and are widened exactly inside the kernels)."""

    def __init__(self, device="cuda:0", dtype=torch.bfloat16):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ShapeError(f"compute dtype {dtype} is neither bfloat16 nor float32")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"this library computes on the GPU only, not on {self.device}")
        self.dtype = dtype
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
            return ops.gemv_bf16(x, w, out_dtype)
        if m <= SKINNY_MAX_ROWS and k % 8 == 0 and k <= SKINNY_MAX_SIDE and w.shape[0] <= SKINNY_MAX_SIDE:
            return ops.gemm_skinny_bf16(x, w, out_dtype)
        return self._library_mm(x, w, out_dtype)

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
