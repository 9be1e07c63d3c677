"""The plain implementation is pinned by what fixes it beside the reference's text: the expected
logits the reference's own fixture holds, the vectors of its unit tests, special cases that reduce to
a library routine, and invariants; each chosen so that a plausible mistake fails it."""
import json
import os

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P

from helpers import reference_fixture

FIXTURE = reference_fixture("tiny-qwen3")
needs_fixture = pytest.mark.skipif(FIXTURE is None, reason="the reference's fixtures are not at hand (RI_REFERENCE_FIXTURES)")


def fixture_model():
    from helpers import read_model_f64
    return read_model_f64(FIXTURE)


@needs_fixture
def test_prefill_logits_equal_the_reference_fixture():
    # tests/model_parity.rs:40-56: logits at every prompt position, bound 2e-4 of the largest + 1e-5
    cfg, w = fixture_model()
    exp = json.load(open(os.path.join(FIXTURE, "expected.json")))
    want = np.fromfile(os.path.join(FIXTURE, "expected_prefill.f32"), dtype="<f4").reshape(len(exp["prompt"]), -1)
    got = P.forward(cfg, w, exp["prompt"])
    assert np.abs(got - want).max() <= 2e-4 * np.abs(want).max() + 1e-5


@needs_fixture
def test_greedy_decode_equals_the_reference_fixture():
    # tests/model_parity.rs:58-68: each decode step's logits and every generated token
    cfg, w = fixture_model()
    exp = json.load(open(os.path.join(FIXTURE, "expected.json")))
    want = np.fromfile(os.path.join(FIXTURE, "expected_decode.f32"), dtype="<f4").reshape(-1, cfg["vocab_size"])
    toks, rows = P.greedy(cfg, w, exp["prompt"], len(exp["generated"]))
    assert toks == exp["generated"]
    for step in range(want.shape[0]):
        assert np.abs(rows[step + 1] - want[step]).max() <= 2e-4 * np.abs(want[step]).max() + 1e-5


def test_rms_norm_vectors_of_the_reference():
    # src/ops/norm.rs:69-81
    x = np.array([[3.0, 4.0, 0.0, 0.0], [1.0, 1.0, 1.0, 1.0]])
    y = P.rms_norm(x, np.ones(4), 0.0)
    assert abs(y[0, 0] - 3.0 / np.sqrt(25.0 / 4.0)) < 1e-12 and abs(y[1, 0] - 1.0) < 1e-12
    h = np.array([2.0, 2.0, 5.0, 5.0]).reshape(2, 2)            # groups of 2
    assert np.allclose(P.rms_norm(h, np.array([1.0, 2.0]), 0.0).reshape(-1), [1.0, 2.0, 1.0, 2.0])


def test_rms_norm_is_the_library_routine_and_eps_sits_inside_the_root():
    rng = np.random.default_rng(0)
    x, g = rng.normal(size=(5, 24)), rng.normal(size=24)
    want = torch.nn.functional.rms_norm(torch.tensor(x), (24,), torch.tensor(g), eps=1e-3).numpy()
    assert np.allclose(P.rms_norm(x, g, 1e-3), want, atol=1e-12)
    # a gain of `1 + w` or eps outside the root would fail the two lines above; scaling invariance at eps 0:
    assert np.allclose(P.rms_norm(7.0 * x, g, 0.0), P.rms_norm(x, g, 0.0))


def test_rope_vectors_of_the_reference():
    # src/ops/rope.rs:86-98: position 0 is the identity; at position 3, theta 1e4, head_dim 4 the pair
    # (element 0, element 2) turns by 3 radians
    x = np.array([1.0, 2.0, 3.0, 4.0]).reshape(1, 1, 4)
    assert np.allclose(P.apply_rope(x, P.rope_angles([0], 4, 1e4)), x)
    y = P.apply_rope(x, P.rope_angles([3], 4, 1e4))[0, 0]
    s3, c3 = np.sin(np.float32(3.0).astype(np.float64)), np.cos(np.float32(3.0).astype(np.float64))
    assert abs(y[0] - (1.0 * c3 - 3.0 * s3)) < 1e-6 and abs(y[2] - (3.0 * c3 + 1.0 * s3)) < 1e-6
    # src/ops/rope.rs:100-111: the norm is kept at position 12345, theta 1e6, head_dim 8
    v = (np.arange(16) - 7.5).reshape(1, 2, 8)
    r = P.apply_rope(v, P.rope_angles([12345], 8, 1e6))
    assert abs((v * v).sum() - (r * r).sum()) < 1e-9


def test_rope_is_a_complex_rotation_of_the_pairs_d_and_d_plus_half():
    rng = np.random.default_rng(1)
    dh, pos = 16, [0, 1, 7, 100]
    x = rng.normal(size=(4, 3, dh))
    inv = P.rope_inv_freq(dh, 1e4).astype(np.float64)
    want = np.empty_like(x)
    for t, p in enumerate(pos):
        z = (x[t, :, :dh // 2] + 1j * x[t, :, dh // 2:]) * np.exp(1j * np.float32(p * inv).astype(np.float64))
        want[t] = np.concatenate([z.real, z.imag], -1)
    # interleaved pairs (2i, 2i+1) or a flipped sign would not give this
    assert np.allclose(P.apply_rope(x, P.rope_angles(pos, dh, 1e4)), want, atol=1e-6)


def test_rope_scores_depend_on_distance_only():
    rng = np.random.default_rng(2)
    q, k = rng.normal(size=(1, 1, 32)), rng.normal(size=(1, 1, 32))

    def score(m, n):
        return (P.apply_rope(q, P.rope_angles([m], 32, 1e4)) * P.apply_rope(k, P.rope_angles([n], 32, 1e4))).sum()
    assert abs(score(9, 4) - score(25, 20)) < 1e-4 and abs(score(9, 4) - score(4, 9)) > 1e-3


def test_inv_freq_is_a_32_bit_power():
    got = P.rope_inv_freq(8, 1e6)
    assert got.dtype == np.float32 and got[0] == 1.0
    assert np.allclose(got, [1.0, 1e6 ** -0.25, 1e6 ** -0.5, 1e6 ** -0.75], rtol=1e-6)


def test_attention_reduces_to_the_library_routine():
    rng = np.random.default_rng(3)
    s, h, hkv, dh = 9, 6, 2, 16
    q, k, v = rng.normal(size=(s, h, dh)), rng.normal(size=(s, hkv, dh)), rng.normal(size=(s, hkv, dh))
    tq = torch.tensor(q).permute(1, 0, 2)[None]
    tk = torch.tensor(k).repeat_interleave(h // hkv, dim=1).permute(1, 0, 2)[None]     # consecutive heads share
    tv = torch.tensor(v).repeat_interleave(h // hkv, dim=1).permute(1, 0, 2)[None]
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)[0].permute(1, 0, 2).numpy()
    assert np.allclose(P.attention(q, k, v), want, atol=1e-10)


def test_attention_special_cases():
    rng = np.random.default_rng(4)
    v = rng.normal(size=(5, 1, 8))
    k = rng.normal(size=(5, 1, 8))
    q = rng.normal(size=(5, 2, 8))
    out = P.attention(q, k, v)
    assert np.allclose(out[0], np.broadcast_to(v[0], (2, 8)))                          # one key: its value
    zero_q = P.attention(np.zeros((5, 1, 8)), k, v)
    assert np.allclose(zero_q[3, 0], v[:4, 0].mean(0))                                 # equal scores: the mean so far
    # the last S of L positions (bottom-right mask): decoding one token sees everything
    assert np.allclose(P.attention(q[4:], k, v)[0], out[4])
    # a window of 2 at position 4 sees keys 3 and 4 only
    w2 = P.attention(q, k, v, window=2)
    assert np.allclose(w2[4], P.attention(q[4:], k[3:], v[3:])[0])


def test_attention_vector_of_the_reference():
    # src/attention.rs:184-219: data sin(0.37 i + seed), 70 positions, head_dim 8, four head groupings,
    # against a dense softmax written here independently
    def data(n, seed):
        return np.sin(np.arange(n, dtype=np.float32) * np.float32(0.37) + np.float32(seed)).astype(np.float64)
    for h, hkv in ((4, 2), (8, 1), (6, 2), (9, 1)):
        total, dh = 70, 8
        k, v = data(total * hkv * dh, 0.1).reshape(total, hkv, dh), data(total * hkv * dh, 0.7).reshape(total, hkv, dh)
        q = data(total * h * dh, 1.3).reshape(total, h, dh)
        got = P.attention(q, k, v)
        for t in (0, 31, 32, 64, 69):
            for hh in range(h):
                kvh = hh // (h // hkv)
                sc = (k[:t + 1, kvh] @ q[t, hh]) / np.sqrt(dh)
                p = np.exp(sc - sc.max())
                assert np.allclose(got[t, hh], (p / p.sum()) @ v[:t + 1, kvh], atol=1e-12)


def test_swiglu_vector_of_the_reference():
    # src/ops/elementwise.rs:59-70: gate [0, 2], up [3, 3] -> [0, 6 / (1 + e^-2)]
    one = np.eye(2)
    y = P.swiglu_mlp(np.array([[0.0, 2.0]]), one, 3.0 * np.ones((2, 2)) / np.array([[0.0 + 2.0]]), one)
    # with x = [0, 2]: gate = x, up = 3 * (x0 + x1) / 2 = 3 for both
    assert abs(y[0, 0]) < 1e-15 and abs(y[0, 1] - 6.0 / (1.0 + np.exp(-2.0))) < 1e-12
    assert np.allclose(P.silu(np.array([0.5])), torch.nn.functional.silu(torch.tensor([0.5], dtype=torch.float64)).numpy())


def test_embedding_and_argmax_vectors():
    table = np.arange(12.0).reshape(4, 3)
    assert np.array_equal(P.embedding(table, [2, 0, 2]), table[[2, 0, 2]])            # src/ops/embedding.rs:49-57
    with pytest.raises(ValueError):
        P.embedding(table, [4])
    assert P.argmax([1.0, 3.0, 3.0]) == 1 and P.argmax([-1.0, 0.0, -5.0]) == 1        # src/ops/reduce.rs:75-78


def test_bf16_rounding_vectors():
    # src/dtype.rs:230-239
    f = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 0.1, -3.25, 65504.0, 1e-20], dtype=np.float32)
    bits = P.f32_to_bf16_bits(f)
    assert list(bits[:3]) == [0x3F80, 0x3F80, 0x3F82]
    want = torch.tensor(f).to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)
    assert np.array_equal(bits, want)
    assert np.isnan(P.bf16_round(np.array([np.nan], dtype=np.float32))[0])


def test_whole_model_with_one_head_and_no_rotation_is_plain_attention():
    # theta so large that every angle beyond pair 0 vanishes does not remove rotation; instead check the
    # layer algebra: with zero attention and feed-forward output matrices the model is embed -> norm -> head
    rng = np.random.default_rng(5)
    cfg = {"vocab_size": 11, "hidden_size": 8, "intermediate_size": 12, "num_hidden_layers": 2,
           "num_attention_heads": 1, "num_key_value_heads": 1, "head_dim": 8, "rms_norm_eps": 1e-6, "rope_theta": 1e4}
    w = {"model.embed_tokens.weight": rng.normal(size=(11, 8)), "model.norm.weight": rng.normal(size=8),
         "lm_head.weight": rng.normal(size=(11, 8))}
    for i in range(2):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = w[p + "post_attention_layernorm.weight"] = np.ones(8)
        for n, shape in (("self_attn.q_proj", (8, 8)), ("self_attn.k_proj", (8, 8)), ("self_attn.v_proj", (8, 8)),
                         ("mlp.gate_proj", (12, 8)), ("mlp.up_proj", (12, 8))):
            w[p + n + ".weight"] = rng.normal(size=shape)
        w[p + "self_attn.o_proj.weight"] = np.zeros((8, 8))
        w[p + "mlp.down_proj.weight"] = np.zeros((8, 12))
        w[p + "self_attn.q_norm.weight"] = w[p + "self_attn.k_norm.weight"] = np.ones(8)
    ids = [3, 1, 4]
    want = P.rms_norm(w["model.embed_tokens.weight"][ids], w["model.norm.weight"], 1e-6) @ w["lm_head.weight"].T
    assert np.allclose(P.forward(cfg, w, ids), want)
    # the attention output is added before the second norm: a non-zero o_proj changes what the feed-forward sees
    w["model.layers.0.self_attn.o_proj.weight"] = rng.normal(size=(8, 8))
    w["model.layers.0.mlp.down_proj.weight"] = rng.normal(size=(8, 12))
    h0 = w["model.embed_tokens.weight"][ids]
    x = P.rms_norm(h0, np.ones(8), 1e-6)
    r = h0 + P.attention_block(x, w, "model.layers.0.self_attn.", cfg, np.arange(3))
    mlp_in = P.rms_norm(r, np.ones(8), 1e-6)
    l0 = r + P.swiglu_mlp(mlp_in, w["model.layers.0.mlp.gate_proj.weight"], w["model.layers.0.mlp.up_proj.weight"],
                          w["model.layers.0.mlp.down_proj.weight"])
    assert np.allclose(P.decoder_layer(h0, w, 0, cfg), l0)


def test_causality_of_the_whole_model(model_dirs):
    from helpers import read_model_f64
    cfg, w = read_model_f64(model_dirs["B"])
    ids = list(np.random.default_rng(6).integers(0, cfg["vocab_size"], 12))
    full = P.forward(cfg, w, ids)
    assert np.allclose(P.forward(cfg, w, ids[:7]), full[:7], atol=1e-9)     # later tokens change nothing earlier
