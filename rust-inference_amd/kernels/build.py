"""Building and loading the HIP kernel library.

The sources under ``csrc/`` are compiled for gfx950 with hipcc into one shared
library beside this file.  ``load()`` takes the library that is there when it was
built from the present sources, and builds it otherwise (in the package folder, or
in a temporary folder when that is not writable), printing a line per file so that
a first call in a fresh checkout shows that it is alive.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

from ..errors import KernelError

ARCH = "gfx950"
LIB_NAME = "libri_kernels.so"
_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")

# -packed-fp32-ops off: packed float32 instructions are not to be generated on this hardware pool
HIPCC_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-Wno-unused-command-line-argument",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# Flags of single files.  The attention kernels take maxima of matrix-core results; unless the compiler may
# take them for numbers, it first passes every operand through an instruction that quiets signalling NaNs
# (IEEE mode), which is a fifth of the softmax's vector instructions.  The kernels produce no NaN from
# numbers: a masked score is -inf, and a column without a key uses 0 as its reference point.
FILE_FLAGS = {"attention_mfma.hip": ["-fno-honor-nans"]}

_lib = None


def _say(msg: str) -> None:
    print(f"[rust-inference_amd] {msg}", file=sys.stderr, flush=True)


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    for path in sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelError("hipcc not found: the HIP kernel library cannot be built")


def _is_current(lib_path: str) -> bool:
    stamp = lib_path + ".hash"
    if not (os.path.exists(lib_path) and os.path.exists(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_hash()


def _compile_one(hipcc: str, src: str, obj: str, env: dict) -> None:
    flags = HIPCC_FLAGS + FILE_FLAGS.get(os.path.basename(src), [])
    proc = subprocess.run([hipcc, *flags, "-c", src, "-o", obj], capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise KernelError(f"hipcc failed on {os.path.basename(src)}:\n{proc.stderr[-4000:]}")


def build(out_dir: str | None = None, jobs: int | None = None) -> str:
    """Compile every source for gfx950 and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = out_dir or _HERE
    os.makedirs(out_dir, exist_ok=True)
    lib_path = os.path.join(out_dir, LIB_NAME)
    srcs = sources()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())          # hipcc wants a HOME for its caches
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    t0 = time.time()
    _say(f"building {LIB_NAME} for {ARCH}: {len(srcs)} files, {jobs} at a time")
    with tempfile.TemporaryDirectory(prefix="ri_build_") as tmp:
        objs = [os.path.join(tmp, os.path.basename(s) + ".o") for s in srcs]
        done = 0

        def one(pair):
            nonlocal done
            _compile_one(hipcc, pair[0], pair[1], env)
            done += 1
            _say(f"  compiled {os.path.basename(pair[0])} ({done}/{len(srcs)}, {time.time() - t0:.0f} s)")

        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(one, zip(srcs, objs)))
        tmp_lib = os.path.join(tmp, LIB_NAME)
        proc = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp_lib],
                              capture_output=True, text=True, env=env)
        if proc.returncode != 0:
            raise KernelError(f"linking {LIB_NAME} failed:\n{proc.stderr[-4000:]}")
        shutil.move(tmp_lib, lib_path + ".tmp")
        os.replace(lib_path + ".tmp", lib_path)
    with open(lib_path + ".hash", "w") as f:
        f.write(source_hash())
    _say(f"built {lib_path} in {time.time() - t0:.0f} s")
    return lib_path


def find_or_build() -> str:
    in_tree = os.path.join(_HERE, LIB_NAME)
    if _is_current(in_tree):
        return in_tree
    if os.access(_HERE, os.W_OK):
        return build(_HERE)
    alt = os.path.join(tempfile.gettempdir(), f"ri_kernels_{os.getuid()}_{source_hash()}")
    alt_lib = os.path.join(alt, LIB_NAME)
    if _is_current(alt_lib):
        return alt_lib
    return build(alt)


# Host-only sources: no kernels in them, so they also build for the host alone (with sanitizers).
HOST_ONLY = ("host_cache.hip", "runtime.hip")


def build_host_sanitized(out_dir: str) -> str:
    """The host-only sources (the cache's bookkeeping, the writer of a step's layout) as a library of their
    own, built for the host alone with the address and undefined-behaviour sanitizers.  For tests on a
    machine without a GPU: the Python process that loads it must have the sanitizer's runtime preloaded
    (``sanitizer_runtime()``), and ``RI_KERNEL_LIBRARY`` tells ``load()`` to take this file."""
    hipcc = _hipcc()
    os.makedirs(out_dir, exist_ok=True)
    lib_path = os.path.join(out_dir, "libri_host_sanitized.so")
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    cmd = [hipcc, "--cuda-host-only", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-fno-omit-frame-pointer",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           *[os.path.join(CSRC, f) for f in HOST_ONLY], "-o", lib_path]
    proc = subprocess.run(cmd, capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise KernelError(f"the sanitized host build failed:\n{proc.stderr[-4000:]}")
    return lib_path


def sanitizer_runtime() -> str:
    """The address sanitizer's shared runtime of the compiler that ``build_host_sanitized`` uses."""
    clang = os.path.join(os.path.dirname(os.path.realpath(_hipcc())), "..", "lib", "llvm", "bin", "clang")
    for cand in (clang, "/opt/rocm/lib/llvm/bin/clang", "/opt/rocm/llvm/bin/clang"):
        if os.path.exists(cand):
            out = subprocess.run([cand, "-print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True, text=True)
            path = out.stdout.strip()
            if out.returncode == 0 and os.path.isabs(path) and os.path.exists(path):
                return path
    raise KernelError("the address sanitizer's runtime library was not found beside the compiler")


# ---- the kernels on the CPU
EMU_LIB_NAME = "libri_emulated.so"
EMU_SRC = os.path.join(CSRC, "emu")


def _rewrite_launches(text: str) -> str:
    """``kernel<...><<<grid, block, shared, stream>>>(args)`` as ``RI_EMU_LAUNCH(kernel<...>, grid, block,
    shared, stream, args)`` and ``extern __shared__ T name[];`` as a pointer to the workgroup's dynamic shared
    memory: what the CPU stand-in of the HIP runtime (csrc/emu) takes instead."""
    import re

    def matching(s: str, at: int, open_ch: str, close_ch: str, step: int) -> int:
        depth, i = 0, at
        while 0 <= i < len(s):
            if s[i] == (open_ch if step > 0 else close_ch):
                depth += 1
            elif s[i] == (close_ch if step > 0 else open_ch):
                depth -= 1
                if depth == 0:
                    return i
            i += step
        raise KernelError("unbalanced brackets around a kernel launch")

    def split_top(s: str) -> list[str]:
        parts, depth, start = [], 0, 0
        for i, ch in enumerate(s):
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "," and depth == 0:
                parts.append(s[start:i])
                start = i + 1
        parts.append(s[start:])
        return [p.strip() for p in parts]

    out, pos = [], 0
    while True:
        at = text.find("<<<", pos)
        if at < 0:
            out.append(text[pos:])
            break
        # the kernel's name, with its template arguments if it has any, stands right before
        begin = at
        if text[begin - 1] == ">":
            begin = matching(text, begin - 1, "<", ">", -1)
        while begin > 0 and (text[begin - 1].isalnum() or text[begin - 1] in "_:"):
            begin -= 1
        close = text.index(">>>", at)
        config = split_top(text[at + 3:close].replace("\\\n", " "))
        while len(config) < 4:
            config.append("0")
        lpar = close + 3
        while text[lpar] in " \\\n\t":
            lpar += 1
        if text[lpar] != "(":
            raise KernelError("a kernel launch without arguments")
        rpar = matching(text, lpar, "(", ")", 1)
        kernel = text[begin:at].strip()
        args = text[lpar + 1:rpar]
        out.append(text[pos:begin])
        out.append(f"RI_EMU_LAUNCH(({kernel}), {config[0]}, {config[1]}, {config[2]}, {config[3]}"
                   + (", " + args if args.strip() else "") + ")")
        pos = rpar + 1
    text = "".join(out)
    return re.sub(r"extern\s+__shared__\s+(\w+)\s+(\w+)\[\];", r"\1* \2 = (\1*)emu::dyn_shared();", text)


def build_emulated(out_dir: str, patches: dict | None = None) -> str:
    """Every kernel source built for the CPU over a stand-in for the HIP runtime (csrc/emu): a workgroup's threads
    run as coroutines that meet at barriers and at every exchange between a wavefront's lanes, so the kernels
    compute what they compute on the GPU, from buffers that the tests lay between guard pages: a load or store
    outside its buffer ends the process with a report.  No GPU is needed.  ``patches``: ``{file: (old, new)}``
    text replacements applied to the copies that are compiled (a test puts a mistake back in to see it caught)."""
    clang = None
    for cand in ("/opt/rocm/llvm/bin/clang++", "/opt/rocm/lib/llvm/bin/clang++", shutil.which("clang++")):
        if cand and os.path.exists(cand):
            clang = cand
            break
    if clang is None:
        raise KernelError("no clang++ for the CPU build of the kernels")
    os.makedirs(out_dir, exist_ok=True)
    lib_path = os.path.join(out_dir, EMU_LIB_NAME)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    gen = os.path.join(out_dir, "emu_src")
    os.makedirs(gen, exist_ok=True)
    for name in os.listdir(CSRC):
        if name.endswith(".h"):
            shutil.copy(os.path.join(CSRC, name), os.path.join(gen, name))
    objs = []
    jobs = []
    for src in sources():
        name = os.path.basename(src)
        with open(src) as f:
            text = f.read()
        if patches and name in patches:
            old, new = patches[name]
            if old not in text:
                raise KernelError(f"{name} does not hold the text to be patched")
            text = text.replace(old, new)
        cpp = os.path.join(gen, name + ".cpp")
        with open(cpp, "w") as f:
            f.write(_rewrite_launches(text))
        obj = cpp + ".o"
        objs.append(obj)
        flags = [f for f in FILE_FLAGS.get(name, [])]
        jobs.append([clang, "-O1", "-g", "-std=c++17", "-fPIC", "-w", "-I", EMU_SRC, "-I", gen, *flags, "-c", cpp, "-o", obj])
    emu_obj = os.path.join(gen, "emu.o")
    jobs.append([clang, "-O1", "-g", "-std=c++17", "-fPIC", "-w", "-I", EMU_SRC, "-c", os.path.join(EMU_SRC, "emu.cpp"),
                 "-o", emu_obj])

    def one(cmd):
        proc = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if proc.returncode != 0:
            raise KernelError(f"the CPU build of {os.path.basename(cmd[-3])} failed:\n{proc.stderr[-6000:]}")

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(one, jobs))
    proc = subprocess.run([clang, "-shared", "-fPIC", *objs, emu_obj, "-o", lib_path], capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise KernelError(f"linking {EMU_LIB_NAME} failed:\n{proc.stderr[-4000:]}")
    return lib_path


PLAIN_LIB_NAME = "libri_plain.so"
PLAIN_SRC = os.path.join(CSRC, "plain")
_plain = None


def _plain_hash() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(PLAIN_SRC)):
        if name.endswith((".cpp", ".h")):
            with open(os.path.join(PLAIN_SRC, name), "rb") as f:
                h.update(name.encode() + f.read())
    return h.hexdigest()[:16]


def build_plain(out_dir: str | None = None) -> str:
    """The plain C++ twins of the kernels (csrc/plain) as a host library of their own; no GPU code in it."""
    out_dir = out_dir or _HERE
    os.makedirs(out_dir, exist_ok=True)
    lib_path = os.path.join(out_dir, PLAIN_LIB_NAME)
    srcs = sorted(os.path.join(PLAIN_SRC, f) for f in os.listdir(PLAIN_SRC) if f.endswith(".cpp"))
    cxx = shutil.which("g++") or shutil.which("c++")
    # no -march: products and sums stay separate instructions, so float32 results are those of the plain text
    cmd = ([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off"] if cxx else
           [_hipcc(), "--cuda-host-only", "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off"])
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.run([*cmd, *srcs, "-o", lib_path + ".tmp"], capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise KernelError(f"building {PLAIN_LIB_NAME} failed:\n{proc.stderr[-4000:]}")
    os.replace(lib_path + ".tmp", lib_path)
    with open(lib_path + ".hash", "w") as f:
        f.write(_plain_hash())
    return lib_path


def load_plain() -> ctypes.CDLL:
    """The plain C++ twins, built at the first call where the library is not there or its sources changed."""
    global _plain
    if _plain is None:
        path = os.path.join(_HERE, PLAIN_LIB_NAME)
        stamp = path + ".hash"
        current = os.path.exists(path) and os.path.exists(stamp) and open(stamp).read().strip() == _plain_hash()
        if not current:
            if os.access(_HERE, os.W_OK):
                path = build_plain(_HERE)
            else:
                alt = os.path.join(tempfile.gettempdir(), f"ri_plain_{os.getuid()}_{_plain_hash()}")
                path = os.path.join(alt, PLAIN_LIB_NAME)
                if not os.path.exists(path):
                    path = build_plain(alt)
        try:
            _plain = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load {path}: {e}") from None
    return _plain


def load() -> ctypes.CDLL:
    """The kernel library, loaded once per process.  Raises KernelError when it
    cannot be had: there is no other implementation to fall back to.  ``RI_KERNEL_LIBRARY``
    names a library to load instead of the one in the tree (a sanitized host build, in tests)."""
    global _lib
    if _lib is None:
        path = os.environ.get("RI_KERNEL_LIBRARY") or find_or_build()
        try:
            _lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load {path}: {e}") from None
        _lib.ri_last_error.restype = ctypes.c_char_p
        _lib.ri_abi_version.restype = ctypes.c_int
    return _lib
