"""The native host code (csrc/host_cache.hip: slots, lengths, page pools, all-or-nothing reservation, the
writer of a step's layout into a pinned buffer) built for the host alone with the address and
undefined-behaviour sanitizers, and the CPU tests that drive it run against that build: an index that
leaves a table, a slot freed twice inside the library or an overflow in its arithmetic ends the run."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cache_and_step_layout_under_sanitizers(tmp_path):
    from rust_inference_amd.errors import KernelError
    from rust_inference_amd.kernels import build
    try:
        lib = build.build_host_sanitized(str(tmp_path))
        runtime = build.sanitizer_runtime()
    except KernelError as e:
        pytest.skip(f"no sanitized build here: {e}")
    env = dict(os.environ, RI_KERNEL_LIBRARY=lib, LD_PRELOAD=runtime,
               ASAN_OPTIONS="detect_leaks=0:halt_on_error=1:abort_on_error=0",
               UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    # the tests of the cache, of the generation loop and of the step layout; the two that ask the attention
    # kernels' host side (not part of this build) stay out
    cmd = [sys.executable, "-m", "pytest", "-q", "-x", "-p", "no:cacheprovider", os.path.join(ROOT, "tests", "test_cache.py"),
           os.path.join(ROOT, "tests", "test_generate_loop.py"), "-k", "not decode_step and not walks_in_runs"]
    run = subprocess.run(cmd, capture_output=True, text=True, env=env, cwd=ROOT, timeout=600)
    assert run.returncode == 0, run.stdout[-3000:] + run.stderr[-3000:]
    assert "passed" in run.stdout and "AddressSanitizer" not in run.stderr and "runtime error" not in run.stderr
    # the run really had the sanitized library: it says so when asked
    probe = subprocess.run([sys.executable, "-c", "from rust_inference_amd.kernels.build import load; import ctypes; "
                            "l = load(); print(l._name); print(hasattr(l, 'ri_argmax'))"],
                           capture_output=True, text=True, env=env, cwd=ROOT, timeout=120)
    assert probe.returncode == 0, probe.stderr[-2000:]
    assert probe.stdout.split() == [lib, "False"]
