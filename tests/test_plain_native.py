"""The plain C++ twins of the kernels (csrc/plain) against the float64 numpy implementation under tests/plain and
the vectors of the reference's own unit tests.  CPU only."""
import numpy as np
import pytest

from plain import qwen3_plain as P
from plain.sampler_plain import PlainRng, PlainSampler
from rust_inference_amd.kernels import plain as N


def rel(got, want):
    want = np.asarray(want, dtype=np.float64)
    return np.abs(np.asarray(got, dtype=np.float64) - want).max() / max(np.abs(want).max(), 1e-30)


def test_bf16_conversion_vectors():
    # src/dtype.rs:230-239: round to nearest even
    assert N.f32_to_bf16(1.0) == 0x3F80 and N.f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80
    assert N.f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82 and N.bf16_to_f32(0x3F80) == 1.0
    assert N.f32_to_bf16(float("nan")) & 0x7FC0 == 0x7FC0
    rng = np.random.default_rng(0)
    for f in rng.normal(size=200).astype(np.float32):
        assert N.f32_to_bf16(f) == int(P.bf16_round(np.array([f], dtype=np.float32)).view(np.uint32)[0] >> 16)


def test_embedding_and_argmax():
    table = np.arange(12, dtype=np.float32).reshape(4, 3)
    assert N.embedding(table, [2, 0, 2]).tolist() == table[[2, 0, 2]].tolist()       # src/ops/embedding.rs:49-57
    with pytest.raises(Exception, match="out of range"):
        N.embedding(table, [4])
    assert N.argmax([1.0, 3.0, 3.0]) == 1 and N.argmax([0.1, 3.0, 2.0]) == 1          # src/ops/reduce.rs:75-78


def test_norms():
    y = N.rms_norm([[3.0, 4.0, 0.0, 0.0], [1.0, 1.0, 1.0, 1.0]], np.ones(4), 0.0)   # src/ops/norm.rs:69-81
    assert abs(y[0, 0] - 3.0 / np.sqrt(25.0 / 4.0)) < 1e-6 and abs(y[1, 0] - 1.0) < 1e-6
    assert np.allclose(N.rms_norm(np.array([2.0, 2.0, 5.0, 5.0]).reshape(2, 2), [1.0, 2.0], 0.0).reshape(-1), [1, 2, 1, 2])
    rng = np.random.default_rng(1)
    x, g, pend = rng.normal(size=(7, 104)), 1 + 0.1 * rng.normal(size=104), rng.normal(size=(7, 104))
    assert rel(N.rms_norm(x, g, 3e-6), P.rms_norm(x, g, 3e-6)) < 2e-6
    total, out = N.add_rms_norm(x, pend, g, 1e-5)
    assert np.array_equal(total, (x.astype(np.float32) + pend.astype(np.float32)))   # src/ops/norm.rs:84-98
    assert rel(out, P.rms_norm(x + pend, g, 1e-5)) < 2e-6
    heads = rng.normal(size=(5, 3, 16))                                                # the per-head form
    assert rel(N.rms_norm(heads, g[:16], 1e-6), P.rms_norm(heads, g[:16], 1e-6)) < 2e-6


def test_rope():
    assert np.allclose(N.rope_inv_freq(48, 5e4), P.rope_inv_freq(48, 5e4), rtol=3e-7, atol=0)
    rng = np.random.default_rng(2)
    x, pos = rng.normal(size=(6, 3, 48)), [0, 1, 5, 100, 1000, 12345]
    # (the table itself within an ulp of the other library's power function; the rotation with the same table,
    # since an ulp of a frequency is a few 1e-4 rad at position 12,345)
    got = N.rope(x, pos, P.rope_inv_freq(48, 5e4))
    assert rel(got, P.apply_rope(x, P.rope_angles(pos, 48, 5e4))) < 3e-6
    assert np.array_equal(got[0], x[0].astype(np.float32))                            # position 0 is the identity
    # src/ops/rope.rs:86-98: position 3, theta 1e4, head_dim 4: the pair (1, 3) turns by 3 * 1e4^(-1/2) rad
    v = N.rope(np.array([[[0.0, 1.0, 0.0, 0.0]]]), [3], N.rope_inv_freq(4, 1e4))[0, 0]
    assert abs(v[1] - np.cos(0.03)) < 1e-6 and abs(v[3] - np.sin(0.03)) < 1e-6
    part = N.rope(x, pos, P.rope_inv_freq(16, 1e4))                                   # a rotation over part of the head
    assert np.array_equal(part[..., 16:], x[..., 16:].astype(np.float32))
    assert rel(part[..., :16], P.apply_rope(x[..., :16], P.rope_angles(pos, 16, 1e4))) < 3e-6


def test_linear_and_swiglu():
    rng = np.random.default_rng(3)
    for m in (1, 2, 3, 4, 5, 9):                                                      # src/cpu/linear.rs:634-647
        x, w = rng.normal(size=(m, 70)), rng.normal(size=(37, 70))
        want = x @ w.T
        assert np.all(np.abs(N.linear(x, w) - want) <= 1e-4 * (1 + np.abs(want)))
    got = N.swiglu([[0.0, 2.0, 3.0, 3.0]])                                            # src/ops/elementwise.rs:59-70
    assert got[0, 0] == 0.0 and abs(got[0, 1] - 6.0 / (1.0 + np.exp(-2.0))) < 1e-6
    y = rng.normal(size=(5, 64)) * 3
    assert rel(N.swiglu(y), P.silu(y[:, :32]) * y[:, 32:]) < 2e-6


@pytest.mark.parametrize("heads, kv_heads", [(4, 2), (8, 1), (6, 2), (9, 1)])       # src/attention.rs:189-219
@pytest.mark.parametrize("window", [None, 20])
def test_paged_attention(heads, kv_heads, window):
    """A 65-token prompt in one go, then five tokens one by one across three pages of 32 (the reference's own
    attention test), pages in a shuffled physical order; head size 8."""
    dh, page = 8, 32
    total = 70
    i = np.arange(total * kv_heads * dh).reshape(total, kv_heads, dh)
    k, v = np.sin(0.37 * i + 1), np.sin(0.37 * i + 2)
    q = np.sin(0.37 * np.arange(total * heads * dh).reshape(total, heads, dh))
    order = [2, 0, 1, 3]
    kp, vp = np.zeros((4, kv_heads, page, dh)), np.zeros((4, kv_heads, dh, page))
    for pos in range(total):
        kp[order[pos // page], :, pos % page] = k[pos]
        vp[order[pos // page], :, :, pos % page] = v[pos]
    table = np.array([order], dtype=np.int32)
    want = P.attention(q, k, v, window=window)
    got = N.attention(q[:65], kp, vp, np.arange(65), np.zeros(65), table, window, 1 / np.sqrt(dh))
    assert rel(got, want[:65]) < 1e-5
    for t in range(65, 70):
        got = N.attention(q[t:t + 1], kp, vp, [t], [0], table, window, 1 / np.sqrt(dh))
        assert rel(got, want[t:t + 1]) < 1e-5


def test_generator_and_sampler_are_the_references():
    a, b = N.Rng(7), PlainRng(7)
    assert a.state == b.state and [a.next_u64() for _ in range(5)] == [b.next_u64() for _ in range(5)]
    assert [N.Rng(0x5EED).next_f32() for _ in range(1)] == [PlainRng(0x5EED).next_f32()]
    rng = np.random.default_rng(4)
    logits = (3 * rng.normal(size=411)).astype(np.float32)
    logits[10] = logits[20]
    history = [int(t) for t in rng.integers(0, 411, 9)]
    for temperature, top_k, top_p, penalty in ((0.0, 0, 1.0, 1.0), (0.0, 0, 1.0, 1.7), (0.8, 0, 1.0, 1.0), (1.3, 5, 1.0, 1.0),
                                               (0.7, 0, 0.8, 1.0), (1.0, 12, 0.6, 1.3), (1.0, 1, 1.0, 1.0)):
        mine, plain = N.Rng(11), PlainSampler(temperature, top_k, top_p, penalty, seed=11)
        for _ in range(40):
            assert N.sample(logits, history, temperature, top_k, top_p, penalty, mine) == plain.sample(logits, history)
    # src/sampling.rs:145-187
    assert N.sample([0.1, 3.0, 2.0], [], 0.0, 0, 1.0, 1.0, N.Rng(1)) == 1
    assert N.sample([0.1, 3.0, 2.0], [1], 0.0, 0, 1.0, 2.0, N.Rng(1)) == 2
    g = N.Rng(7)
    picks = [N.sample([0.0, float(np.log(3.0))], [], 1.0, 0, 1.0, 1.0, g) for _ in range(4000)]
    assert abs(np.mean(picks) - 0.75) < 0.03
    g = N.Rng(3)
    assert {N.sample([3.0, 1.0, 0.5, 0.0], [], 1.0, 0, 0.5, 1.0, g) for _ in range(50)} == {0}
