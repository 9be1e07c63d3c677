"""The kernels without a GPU: every kernel source compiled for the CPU (kernels/build.py: build_emulated; a
workgroup's threads are coroutines that meet at barriers and at every exchange between the lanes of a wavefront,
the matrix-core product included) and run by the kernel tests themselves, tests/test_kernels_gpu.py, with every
operand and every buffer the wrappers allocate between two guard pages.  The kernels keep their loads out of
branches and issue them whatever the indices are, from addresses pulled back inside the data: here an address
that was not pulled back far enough touches a guard page and ends the run with a report that names the kernel,
the workgroup, the thread and the buffer.  The sizes are the GPU tests' own except the largest (the emulation
runs a few thousand matrix instructions a second)."""
import os
import subprocess
import sys
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HERE = os.path.join(ROOT, "tests")

# What stays out: matrices of 4,096 and more rows or columns, contexts of thousands of keys and steps of hundreds of
# (sequence, kv head) pairs (minutes each when emulated); every kernel and every form of it is still run, at the
# smaller sizes of the same tests or, where the form is chosen by the machine's size, on a machine made small (below).
SELECT = ("not 4096 and not 12288 and not 5120 and not 5000 and not very_long and not more_pages_than and not thousands "
          "and not (many_sequences and not (16-8-32-100 or 16-8-32-40)) and not (in_runs and not 8-8-32) "
          "and not (wide_packed and 1000 and not (1000-1024-33 or 1000-1024-64)) and not eight_wavefronts")


def _env(extra=None):
    env = dict(os.environ, RI_TEST_KERNELS="emulated", **(extra or {}))
    env.pop("RI_KERNEL_LIBRARY", None)
    return env


def _run(args, env_extra=None, timeout=1500):
    return subprocess.run([sys.executable, *args], capture_output=True, text=True, env=_env(env_extra), cwd=ROOT,
                          timeout=timeout)


def _start(args, env_extra=None):
    """The same in the background, its output in files (a pipe that fills up would stop it)."""
    out, err = tempfile.TemporaryFile("w+"), tempfile.TemporaryFile("w+")
    return subprocess.Popen([sys.executable, *args], stdout=out, stderr=err, text=True, env=_env(env_extra), cwd=ROOT), out, err


def _workers(most):
    """A few processes side by side where the plugin for that is installed."""
    try:
        import xdist  # noqa: F401
        return ["-n", str(max(1, min(most, (os.cpu_count() or 2) // 2)))]
    except ImportError:
        return []


# With one compute unit every launch "fills the machine": the prompt attention keeps its tiles of 32 and 64 rows a
# wavefront (on 256 units the small cases all run with the smallest), and the wide product plans for one unit.
ONE_UNIT = ("one_run or mfma_prefill_attention or (mfma_attention_window_edges and prefill) or "
            "(mfma_attention_finds_one_far_key and prefill) or (wide_packed and not 4096 and not 12288 and not 5120 "
            "and not (1000 and not (1000-1024-33 or 1000-1024-64)))")
PYTEST = ["-m", "pytest", "-q", "-x", "-p", "no:cacheprovider"]
KERNEL_TESTS, SMALL_MACHINE = os.path.join(HERE, "test_kernels_gpu.py"), os.path.join(HERE, "small_machine_kernels.py")
SAMPLER_TESTS = os.path.join(HERE, "test_sampling_gpu.py")
SAMPLER_SELECT = "(same_token_as_the_plain_sampler or top_p_drops) and not large"     # not the 151,936 entries, not the engine


@pytest.fixture(scope="module")
def runs():
    """The four emulated runs, side by side (each is a pytest of its own; together they take what the longest takes)."""
    from rust_inference_amd.errors import KernelError
    try:
        sys.path.insert(0, HERE)
        import emulated
        emulated.library()
    except KernelError as e:
        pytest.skip(f"no CPU build of the kernels here: {e}")
    started = {
        "kernel tests": _start([*PYTEST, *_workers(4), KERNEL_TESTS, "-k", SELECT]),
        "sixteen units": _start([*PYTEST, SMALL_MACHINE], {"RI_EMU_COMPUTE_UNITS": "16"}),
        "one unit": _start([*PYTEST, *_workers(2), SMALL_MACHINE, KERNEL_TESTS, "-k", ONE_UNIT], {"RI_EMU_COMPUTE_UNITS": "1"}),
        "sampler": _start([*PYTEST, *_workers(2), SAMPLER_TESTS, "-k", SAMPLER_SELECT]),
    }
    done = {}
    try:
        for name, (proc, out, err) in started.items():
            proc.wait(timeout=1500)
            out.seek(0), err.seek(0)
            done[name] = (proc.returncode, out.read(), err.read())
    finally:
        for proc, out, err in started.values():
            if proc.poll() is None:
                proc.kill()
            out.close(), err.close()
    return done


def _passed(run, tests=None):
    code, out, err = run
    assert code == 0, out[-3000:] + err[-3000:]
    assert (f"{tests} passed" if tests else " passed") in out and "[emu]" not in err, out[-2000:]


def test_the_kernel_tests_pass_on_the_cpu_build_between_guard_pages(runs):
    _passed(runs["kernel tests"])


def test_the_sampler_tests_pass_on_the_cpu_build_between_guard_pages(runs):
    _passed(runs["sampler"], 33)


@pytest.mark.parametrize("units, tests", [("sixteen units", 7), ("one unit", 61)])
def test_the_forms_that_a_large_step_chooses_on_a_machine_made_small(runs, units, tests):
    """tests/small_machine_kernels.py: the emulated runtime reports a few compute units, so that the walk in runs, the
    joins of many pieces and the run of more than 1,024 pages are chosen for one or two heads; with one unit also
    the kernel tests whose launches are sized by the machine."""
    _passed(runs[units], tests)


# The product for 17 to 64 rows once read a tile of x that its buffer does not have (33 to 48 rows were three
# tiles of 16 and ran with code built for four; the loads that are issued whatever the indices are read the
# fourth): a kilobyte per step past the end of the buffer, which on the GPU faulted once in many runs.  The
# address is pulled back to the last tile now (and 33 to 48 rows have code for three); the kernel still runs with
# more tiles than x has where a step of up to 16 rows takes it, and with the old expression put back such a run
# must end at the guard page and say where.
OLD_MID = {"gemm_skinny_bf16.hip": ("min(rt, (M - 1) >> 4)", "rt")}
PROBE = """
import sys
sys.path.insert(0, {here!r})
import torch, emulated
ops = emulated.ops(patches={patches!r})
m, n, k = 10, 48, 1024
w = (torch.randn(n, k) * 0.1).bfloat16()
x = ops.TiledRows.empty(m, k, "cpu")
x.data.zero_()
ops.gemm_mid_packed_bf16(x, emulated.tensor(ops.pack_for_mfma(w), "packed weights"), n, torch.float32)
print("no access outside a buffer")
"""


def test_a_load_that_leaves_its_buffer_is_caught_and_named():
    from rust_inference_amd.errors import KernelError
    try:
        sys.path.insert(0, HERE)
        import emulated
        emulated.library(OLD_MID)
    except KernelError as e:
        pytest.skip(f"no CPU build of the kernels here: {e}")
    bad = _run(["-c", PROBE.format(here=HERE, patches=OLD_MID)])
    assert bad.returncode == 86, bad.stdout[-2000:] + bad.stderr[-2000:]
    assert "gemm_mid_packed_kernel" in bad.stderr and "past the end of buffer" in bad.stderr
    good = _run(["-c", PROBE.format(here=HERE, patches=None)])
    assert good.returncode == 0 and "no access outside a buffer" in good.stdout, good.stdout[-2000:] + good.stderr[-2000:]
