"""The argmax entry point that allocates nothing, called through ctypes as a caller without an allocator
would: two calls in a row on one GPU, the second with a smaller input, each against ``ri_argmax``."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_argmax_static_matches_argmax_on_two_calls_in_a_row():
    from rust_inference_amd.kernels import ops
    from rust_inference_amd.kernels.build import load

    lib = load()
    lib.ri_argmax_static.restype = ctypes.c_int
    lib.ri_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.ri_argmax_static_max_rows.restype = ctypes.c_int
    lib.ri_last_error.restype = ctypes.c_char_p
    assert lib.ri_argmax_static_max_rows() == 1024

    # Free device memory as the driver counts it: an allocation inside the entry point (which torch's own counter
    # would not see) takes at least a page of it.  The first call on a device looks up the built-in array's
    # address, so one untimed call comes first and the comparison is made on the calls after it.
    hip = ctypes.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    dev = torch.device("cuda:0")
    gen = torch.Generator(device="cpu").manual_seed(11)
    stream = torch.cuda.current_stream(dev).cuda_stream
    # the second call is smaller in rows and in width: what the first left in the array must not show
    warm = torch.zeros((2, 64), dtype=torch.float32, device=dev)
    warm_out = torch.zeros(2, dtype=torch.int32, device=dev)
    assert lib.ri_argmax_static(warm_out.data_ptr(), warm.data_ptr(), 2, 64, stream) == 0
    torch.cuda.synchronize()
    for rows, vocab in ((37, 151936), (5, 1000)):
        logits = torch.randn((rows, vocab), generator=gen, dtype=torch.float32).to(dev)
        logits[1, 7] = logits[1, vocab - 3] = 99.0          # a tie: the lower index wins
        want = ops.argmax(logits)
        got = torch.full((rows,), -1, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(dev), free_bytes()
        rc = lib.ri_argmax_static(got.data_ptr(), logits.data_ptr(), rows, vocab, stream)
        assert rc == 0, lib.ri_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == before
        # (the workspace this entry point spares is half a megabyte: an allocation of it could not hide in less)
        assert free_before - free_bytes() < 256 * 1024, "the driver's free memory shrank across the call"
        assert torch.equal(got, want), (rows, vocab)
        assert got[1].item() == 7
        assert torch.equal(got.cpu().long(), logits.cpu().argmax(1))

    # more rows than the built-in array holds: refused with a reason, nothing launched
    rows = lib.ri_argmax_static_max_rows() + 1
    logits = torch.zeros((rows, 8), dtype=torch.float32, device=dev)
    got = torch.full((rows,), -1, dtype=torch.int32, device=dev)
    assert lib.ri_argmax_static(got.data_ptr(), logits.data_ptr(), rows, 8, stream) != 0
    assert "1024" in lib.ri_last_error().decode()
    torch.cuda.synchronize()
    assert int(got.max()) == -1
