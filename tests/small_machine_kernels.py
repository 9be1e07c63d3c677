"""Kernel tests for the CPU build of the kernels alone (tests/test_kernels_emulated.py runs this file; pytest does
not collect it by itself).  Some forms of the decode attention are chosen by the size of the step against the size
of the machine: a sequence walked in several runs that are joined afterwards from 16,384 keys on where the step
does not fill the compute units, one run of more than 1,024 pages, a join of more than sixteen pieces.  On an MI355X
those take tens of thousands of keys over several heads, minutes each when emulated.  Here the emulated runtime
says it has RI_EMU_COMPUTE_UNITS compute units (16, or 1 for the test that says so), the rules choose the same forms
for one or two heads, and every load of theirs that is issued whatever the indices are runs between guard pages."""
import numpy as np
import pytest
import torch

from test_kernels_gpu import (BF16_OUT, EMULATED, attention_case, close, f64, fused_decode_case, ops, t,  # noqa: F401
                              _guarded_buffers_go_back)

if not EMULATED:
    pytest.skip("for the CPU build of the kernels", allow_module_level=True)


def far_key(seq, kv_head, head, dh, far):
    def boost(qkv, k, kp, table):
        kf = f64(kp[table[seq, far // 32].item(), kv_head, far % 32])
        qkv[seq, head * dh:(head + 1) * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
    return boost


def machine(ops, units):
    if ops.compute_units() != units:
        pytest.skip(f"runs where the emulated machine has {units} compute units")


def test_long_sequences_in_runs_that_are_joined(ops):
    """Three sequences of two kv heads, one of 16,400 keys: eight runs each, cut by each sequence's own length
    (most of a short one's are empty); a key that stands out in the first run and one in the last."""
    machine(ops, 16)
    heads, kv_heads, dh, lens = 2, 2, 32, [16400, 700, 33]
    assert ops.decode_attention_runs(len(lens), kv_heads, max(lens) + 300) == 8
    for far in (3, 16000):
        out, want = attention_case(ops, np.random.default_rng(far), lens, [1] * len(lens), heads, kv_heads, dh,
                                   torch.bfloat16, boost=far_key(0, 1, 1, dh, far), kernel="decode")
        close(out, want, BF16_OUT, f"runs, far key {far}")


def test_long_sequences_in_runs_from_the_raw_projection(ops):
    """The same walk by the kernel that norms and rotates q and k and stores the new key and value first."""
    machine(ops, 16)
    lens = [16400, 700, 33]
    assert ops.decode_attention_runs(len(lens), 2, max(lens) + 301) == 8
    fused_decode_case(ops, 4, 2, 32, None, lens, steps=1, repeats=1)


def test_more_than_sixteen_runs_are_joined_in_groups(ops):
    """One sequence of 35,000 keys beside a short one: 17 runs each, joined in eight groups side by side."""
    machine(ops, 16)
    heads, kv_heads, dh, lens = 1, 1, 32, [35000, 300]
    assert ops.decode_attention_runs(len(lens), kv_heads, max(lens) + 300) == 17
    for far in (100, 34990):
        out, want = attention_case(ops, np.random.default_rng(far), lens, [1] * len(lens), heads, kv_heads, dh,
                                   torch.bfloat16, boost=far_key(0, 0, 0, dh, far), kernel="decode")
        close(out, want, BF16_OUT, f"17 runs, far key {far}")


def test_more_than_sixteen_chunks_are_joined_in_runs(ops):
    """The kernel of one workgroup per chunk of 256 keys, past 16 chunks a sequence, with a window too."""
    machine(ops, 16)
    heads, kv_heads, dh, lens = 2, 1, 32, [4097, 6000, 700]
    assert ops.decode_attention_runs(len(lens), kv_heads, max(lens) + 300) == 0
    for far, window in ((0, None), (5999, None), (5000, 4500)):
        out, want = attention_case(ops, np.random.default_rng(far), lens, [1] * len(lens), heads, kv_heads, dh,
                                   torch.bfloat16, window=window, boost=far_key(1, 0, 1, dh, far), kernel="decode")
        close(out, want, BF16_OUT, f"chunks, far key {far}, window {window}")


@pytest.mark.parametrize("heads, kv_heads, dh, window", [(16, 8, 32, None), (8, 8, 64, 100), (128, 8, 64, None)])
def test_one_run_for_every_compute_unit_walks_with_eight_wavefronts(ops, heads, kv_heads, dh, window):
    """Two sequences of eight kv heads on sixteen compute units: a run for each, walked by eight wavefronts, from
    the normed queries and from the raw projection (sixteen query heads a kv head: two for a wavefront to norm)."""
    machine(ops, 16)
    lens = [1200, 33]
    assert ops.decode_attention_runs(2, kv_heads, max(lens) + 301) == 1      # (too few pairs for the walk by four)
    assert ops.decode_attention_runs(3, kv_heads, max(lens) + 301) == 0
    if heads <= 16:
        out, want = attention_case(ops, np.random.default_rng(dh), lens, [1, 1], heads, kv_heads, dh, torch.bfloat16,
                                   window=window, boost=far_key(0, 3, 3 * (heads // kv_heads), dh, 40), kernel="decode")
        close(out, want, BF16_OUT, f"eight wavefronts a run, window {window}")
    fused_decode_case(ops, heads, kv_heads, dh, window, lens, steps=2, repeats=1)


def test_one_run_of_more_pages_than_a_wavefront_holds_table_entries_for(ops):
    """A wavefront fetches the table's entries for 256 of its pages at a time; in one run of more than 1,024
    pages it goes round that loop again.  Two sequences on a machine of one compute unit: one run each."""
    machine(ops, 1)
    heads, kv_heads, dh, lens = 1, 1, 32, [33100, 32800]
    assert ops.decode_attention_runs(len(lens), kv_heads, max(lens) + 300) == 1
    for far in (9000, 33000):
        out, want = attention_case(ops, np.random.default_rng(far), lens, [1] * len(lens), heads, kv_heads, dh,
                                   torch.bfloat16, boost=far_key(0, 0, 0, dh, far), kernel="decode")
        close(out, want, BF16_OUT, f"one long run, far key {far}")
