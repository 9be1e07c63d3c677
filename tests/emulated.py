"""The kernels on the CPU, for tests without a GPU: `rust_inference_amd.kernels.ops` as it is, over the library
that `kernels/build.py: build_emulated` makes (every kernel source compiled for the host over a stand-in for the
HIP runtime), with every tensor the wrappers are given or allocate laid between two guard pages.  A kernel that
reads or writes outside a buffer ends the process with a report (exit status 86), one whose threads wait for
one another for ever with status 87: run what uses this in a process of its own.

    ops = emulated.ops()                      # builds the library at the first call (a minute), then loads it
    x = emulated.tensor(torch_cpu_tensor)     # a copy between guard pages, its end against the page behind it
"""
import ctypes
import hashlib
import os
import sys
import tempfile

import torch

_state = {}


def library(patches=None) -> str:
    """Path of the emulated library for the present sources (and patches), built where it is not there yet."""
    from rust_inference_amd.kernels import build
    h = hashlib.sha256(build.source_hash().encode())
    for name in sorted(os.listdir(build.EMU_SRC)):
        path = os.path.join(build.EMU_SRC, name)
        for root, _, files in os.walk(path) if os.path.isdir(path) else [(os.path.dirname(path), [], [name])]:
            for f in sorted(files):
                with open(os.path.join(root, f), "rb") as fh:
                    h.update(f.encode() + fh.read())
    h.update(repr(sorted((patches or {}).items())).encode())
    out = os.path.join(tempfile.gettempdir(), f"ri_emulated_{os.getuid()}_{h.hexdigest()[:16]}")
    lib = os.path.join(out, build.EMU_LIB_NAME)
    if not os.path.exists(lib):
        print(f"[emulated] building the kernels for the CPU in {out}", file=sys.stderr, flush=True)
        tmp = out + f".{os.getpid()}"
        build.build_emulated(tmp, patches)
        try:
            os.rename(tmp, out)
        except OSError:                       # another process was faster
            pass
    return lib


def tensor(t: torch.Tensor, name: str = "input", flush_end: bool = True) -> torch.Tensor:
    """A copy of a CPU tensor in guarded memory."""
    g = empty(tuple(t.shape), t.dtype, name, flush_end)
    g.copy_(t)
    return g


def empty(shape, dtype, name="buffer", flush_end=True) -> torch.Tensor:
    lib = _state["lib"]
    shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list, torch.Size)) else (shape,)))
    numel = 1
    for s in shape:
        numel *= s
    nbytes = numel * torch.empty((), dtype=dtype).element_size()
    ptr = lib.ri_emu_alloc(max(nbytes, 16), int(flush_end), name.encode())
    if not ptr:
        raise MemoryError(f"no guarded buffer of {nbytes} bytes")
    # (sizes are rounded up to 16 bytes, so that every buffer starts as aligned as an allocation on the GPU does
    # and the kernels choose the loads they choose there: up to 15 bytes behind an odd-sized buffer go unseen)
    if numel == 0:
        return torch.empty(shape, dtype=dtype)
    buf = (ctypes.c_ubyte * nbytes).from_address(ptr)
    return torch.frombuffer(buf, dtype=dtype, count=numel).view(shape)


class _Torch:
    """`torch` for the wrappers: what they allocate lies between guard pages."""

    def __getattr__(self, name):
        return getattr(torch, name)

    @staticmethod
    def empty(*shape, dtype=torch.float32, device=None, **kw):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list, torch.Size)):
            shape = shape[0]
        return empty(shape, dtype, "allocated by the wrapper")

    @staticmethod
    def zeros(*shape, dtype=torch.float32, device=None, **kw):
        return _Torch.empty(*shape, dtype=dtype).zero_()

    @staticmethod
    def full(shape, value, dtype=torch.float32, device=None, **kw):
        return _Torch.empty(shape, dtype=dtype).fill_(value)


def ops(patches=None):
    """`rust_inference_amd.kernels.ops` running on the CPU.  Once per process."""
    if "ops" in _state:
        return _state["ops"]
    os.environ["RI_KERNEL_LIBRARY"] = library(patches)
    from rust_inference_amd.errors import ShapeError
    from rust_inference_amd.kernels import build, ops as real
    lib = build.load()
    lib.ri_emu_alloc.restype = ctypes.c_void_p
    lib.ri_emu_alloc.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_char_p]
    _state["lib"] = lib

    def dev(t, name, dtype=None, shape=None):
        if not isinstance(t, torch.Tensor) or t.is_cuda:
            raise TypeError(f"{name}: the emulated kernels take CPU tensors")
        if not t.is_contiguous():
            raise ShapeError(f"{name} must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise ShapeError(f"{name} must be {dtype}, got {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise ShapeError(f"{name} must have shape {list(shape)}, got {list(t.shape)}")
        return t.data_ptr()

    real._dev = dev
    real._stream = lambda: 0
    real.torch = _Torch()
    _state["ops"] = real
    return real


def free_all():
    _state["lib"].ri_emu_free_all()
