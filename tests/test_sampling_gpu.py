"""The device sampler against the plain sampler: the same logits and the same uniform draw give the same token.

The kernel tests of this file also run without a GPU, on the CPU build of the kernels between guard pages, when
the environment says RI_TEST_KERNELS=emulated (tests/test_kernels_emulated.py starts that run)."""
import os

import numpy as np
import pytest
import torch

from plain.sampler_plain import PlainRng, argmax, candidates, draw, penalise

EMULATED = os.environ.get("RI_TEST_KERNELS") == "emulated"
pytestmark = [] if EMULATED else pytest.mark.gpu
DEV = "cpu" if EMULATED else "cuda:0"


@pytest.fixture(scope="module")
def ops():
    if EMULATED:
        import emulated
        return emulated.ops()
    from rust_inference_amd.kernels import ops
    return ops


@pytest.fixture(autouse=True)
def _guarded_buffers_go_back():
    yield
    if EMULATED:
        import gc
        import emulated
        gc.collect()
        emulated.free_all()


def g(x):
    """On the GPU the tensor itself; emulated, a copy between guard pages."""
    if EMULATED:
        import emulated
        return emulated.tensor(x.contiguous(), "a test's operand")
    return x


def plain_pick(logits, r, temperature, top_k, top_p, penalty, history):
    row = penalise(logits, history, penalty)
    if temperature <= 0:
        return argmax(row)
    order, probs = candidates(row, temperature, top_k, top_p)
    return draw(order, probs, r)


@pytest.mark.parametrize("temperature, top_k, top_p, penalty", [
    (0.8, 0, 1.0, 1.0), (1.3, 5, 1.0, 1.0), (0.7, 0, 0.8, 1.0), (1.0, 12, 0.6, 1.3), (0.0, 0, 1.0, 1.7),
    (1.0, 1, 1.0, 1.0), (0.5, 0, 0.05, 1.0), (2.0, 400, 0.999, 1.0),
])
@pytest.mark.parametrize("split", [False, True])                 # a workgroup a row; a row over many workgroups
@pytest.mark.parametrize("vocab", [411, 4096])                  # no power of two; and rows read 16 bytes at a time,
def test_same_token_as_the_plain_sampler(ops, temperature, top_k, top_p, penalty, vocab, split):   # more ties than are listed
    rng = np.random.default_rng(int(temperature * 10) + top_k)
    rows = 24
    logits = (3.0 * rng.normal(size=(rows, vocab))).astype(np.float32)
    logits[:, 10] = logits[:, 20]                               # ties inside every row
    logits[3, :] = 0.25                                         # a row of equal logits: the id order decides alone
    logits[4, 100:300] = logits[4, 100]
    history = [[int(t) for t in rng.integers(0, vocab, 9)] for _ in range(rows)]
    gen = PlainRng(5)
    rs = [gen.next_f32() for _ in range(rows)]
    rs[0], rs[1] = 0.0, float(np.float32(1.0) - np.float32(2.0 ** -24))   # the ends of [0, 1)
    seen = g(torch.zeros((rows, vocab), dtype=torch.uint8, device=DEV))
    hr = [r for r in range(rows) for _ in history[r]]
    ht = [t for r in range(rows) for t in history[r]]
    ops.mark_seen(seen, g(torch.tensor(hr, dtype=torch.int32, device=DEV)), g(torch.tensor(ht, dtype=torch.int32, device=DEV)))
    got = ops.sample(g(torch.tensor(logits, device=DEV)), g(torch.tensor(rs, dtype=torch.float32, device=DEV)), temperature,
                     top_k, top_p, penalty, seen if penalty != 1.0 else None, split=split).tolist()
    want = [plain_pick(logits[r], rs[r], temperature, top_k, top_p, penalty, history[r]) for r in range(rows)]
    # the device sums masses exactly, the plain sampler in float32 in drawing order: a draw that falls within
    # float32 rounding of a boundary may land on the neighbour; allow that for at most one row, and only then
    wrong = [r for r in range(rows) if got[r] != want[r]]
    for r in wrong:
        order, probs = candidates(penalise(logits[r], history[r], penalty), temperature, top_k, top_p)
        acc = np.cumsum(probs.astype(np.float64))
        assert np.min(np.abs(acc - rs[r])) < 1e-5, f"row {r}: {got[r]} against {want[r]} away from any boundary"
    assert len(wrong) <= 1


def test_large_vocabulary_and_distribution(ops):
    """151,936 entries; 4,000 draws from two dominant tokens follow their probabilities (src/sampling.rs:167-177)."""
    vocab = 151936
    logits = torch.full((1, vocab), -30.0, device=DEV)
    logits[0, 1000], logits[0, 150000] = 0.0, float(np.log(3.0))
    gen = PlainRng(7)
    rs = g(torch.tensor([gen.next_f32() for _ in range(4000)], dtype=torch.float32, device=DEV))
    picks = ops.sample(logits.expand(4000, vocab).contiguous(), rs, 1.0).tolist()
    assert set(picks) <= {1000, 150000}
    assert abs(np.mean([p == 150000 for p in picks]) - 0.75) < 0.03
    again = ops.sample(logits.expand(4000, vocab).contiguous(), rs, 1.0).tolist()
    assert picks == again                                         # the same draws, the same tokens
    assert picks == ops.sample(logits.expand(4000, vocab).contiguous(), rs, 1.0, split=False).tolist()


def test_both_forms_pick_the_same_tokens_of_a_large_vocabulary(ops):
    """Logits like a model's over 151,936 entries, with ties, penalty, top-k and top-p: the row cut over many
    workgroups gives the token that the single workgroup gives, and a few rows are checked against the
    plain sampler."""
    rng = np.random.default_rng(11)
    vocab, rows = 151936, 16
    logits = (2.5 * rng.normal(size=(rows, vocab))).astype(np.float32)
    logits[:, 5000:5400] = logits[:, 5000:5001]                  # 400 tied candidates in every row
    logits[2, :] = 1.5                                           # more ties than are listed
    logits[3, 70000] = 30.0                                      # one token owns the row
    history = [[int(t) for t in rng.integers(0, vocab, 50)] for _ in range(rows)]
    seen = g(torch.zeros((rows, vocab), dtype=torch.uint8, device=DEV))
    ops.mark_seen(seen, g(torch.tensor([r for r in range(rows) for _ in history[r]], dtype=torch.int32, device=DEV)),
                  g(torch.tensor([t for r in range(rows) for t in history[r]], dtype=torch.int32, device=DEV)))
    gen = PlainRng(3)
    rs = [gen.next_f32() for _ in range(rows)]
    dl, dr = g(torch.tensor(logits, device=DEV)), g(torch.tensor(rs, dtype=torch.float32, device=DEV))
    # (47 kept of a row of equal logits: 0.9 of them is no whole number, so float32 sums cannot sit on the edge)
    for temperature, top_k, top_p, penalty in ((0.8, 0, 1.0, 1.0), (1.0, 47, 0.9, 1.2), (1.5, 0, 0.95, 1.0),
                                               (0.7, 3000, 1.0, 1.1)):
        sn = seen if penalty != 1.0 else None
        one = ops.sample(dl, dr, temperature, top_k, top_p, penalty, sn, split=False).tolist()
        many = ops.sample(dl, dr, temperature, top_k, top_p, penalty, sn, split=True).tolist()
        assert one == many, (temperature, top_k, top_p, penalty)
        for r in (0, 2, 3):
            want = plain_pick(logits[r], rs[r], temperature, top_k, top_p, penalty, history[r])
            if many[r] != want:                                   # only within float32 rounding of a boundary
                order, probs = candidates(penalise(logits[r], history[r], penalty), temperature, top_k, top_p)
                assert np.min(np.abs(np.cumsum(probs.astype(np.float64)) - rs[r])) < 1e-5, (r, many[r], want)


def test_top_p_drops_the_tail_and_top_k_one_is_greedy(ops):
    row = g(torch.tensor([[3.0, 1.0, 0.5, 0.0]], device=DEV).expand(50, 4).contiguous())
    rs = g(torch.linspace(0, 0.999, 50, device=DEV))
    assert set(ops.sample(row, rs, 1.0, top_p=0.5).tolist()) == {0}              # src/sampling.rs:179-187
    row = g(torch.tensor([[0.5, 0.4, 0.6, 0.1]], device=DEV).expand(50, 4).contiguous())
    assert set(ops.sample(row, rs, 1.0, top_k=1).tolist()) == {2}                # src/sampling.rs:157-164
    assert ops.sample(g(torch.tensor([[0.1, 3.0, 2.0]], device=DEV)), None, 0.0).tolist() == [1]
    seen = g(torch.zeros((1, 3), dtype=torch.uint8, device=DEV))
    seen[0, 1] = 1
    assert ops.sample(g(torch.tensor([[0.1, 3.0, 2.0]], device=DEV)), None, 0.0, penalty=2.0, seen=seen).tolist() == [2]


def test_generation_with_penalty_and_temperature_is_seeded(model_dirs):
    from rust_inference_amd import Model
    model = Model.load(model_dirs["A"], dtype="float32", max_batch=3, max_seq_len=64)
    prompts = [[1, 2, 3, 4], [9, 8], [5]]
    kw = dict(max_new_tokens=10, temperature=0.9, top_k=40, top_p=0.95, repetition_penalty=1.2)
    a = model.generate(prompts, seed=3, **kw).tokens
    b = model.generate(prompts, seed=3, **kw).tokens
    alone = model.generate(prompts[:1], seed=3, **kw).tokens
    assert a == b and alone[0] == a[0] and a != model.generate(prompts, seed=4, **kw).tokens


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_repetition_penalty_gives_the_same_tokens_with_the_loop_running_ahead(model_dirs, dtype_name):
    """With graphs the loop launches a step before it has read the ids of the one before, and marks the penalty's
    history on the device from the ids in flight; without, the host marks it from the ids it has read.  The same
    tokens either way (the steps are the same kernels on the same rows as long as nobody stops), with stop tokens
    too in float32 (a sequence that stops is carried one step further by the one loop; nobody else's logits
    change for that in 32-bit)."""
    from rust_inference_amd import Model
    prompts = [[1, 2, 3, 4, 2, 2], [9, 8], [5], [7, 7, 7, 7]]
    kw = dict(max_new_tokens=24, temperature=0.9, top_k=30, repetition_penalty=1.4, seed=11)
    outs = {}
    for graphs in (True, False):
        model = Model.load(model_dirs["A"], dtype=dtype_name, max_batch=4, max_seq_len=64, use_graphs=graphs, graph_after=0)
        outs[graphs] = [model.generate(prompts, ignore_eos=True, **kw)]
        if dtype_name == "float32":
            outs[graphs].append(model.generate(prompts, stop_token_ids=[int(t) for t in outs[graphs][0].tokens[1][3:9]], **kw))
        model.cache.check_consistent()
    for a, b in zip(outs[True], outs[False]):
        assert a.tokens == b.tokens and a.finish_reasons == b.finish_reasons
    if dtype_name == "float32":
        assert "stop" in outs[True][1].finish_reasons
    plain = Model.load(model_dirs["A"], dtype=dtype_name, max_batch=4, max_seq_len=64, use_graphs=True, graph_after=0)
    assert plain.generate(prompts, ignore_eos=True, **dict(kw, repetition_penalty=1.0)).tokens != outs[True][0].tokens


def test_sequences_of_one_batch_sample_each_in_their_own_way(model_dirs):
    """Per-request sampling parameters through the entry point: greedy, temperature, top-k with a penalty side
    by side in one batch give each request the tokens it gets when the whole batch samples its way (float32:
    a request's logits do not depend on its neighbours; its generator is seeded by its index either way)."""
    from rust_inference_amd import Model
    from rust_inference_amd.sampling import SamplingParams
    model = Model.load(model_dirs["A"], dtype="float32", max_batch=4, max_seq_len=64)
    prompts = [[1, 2, 3, 4], [9, 8], [5], [7, 7, 7]]
    kinds = [SamplingParams(), SamplingParams(temperature=0.9, seed=3), SamplingParams(temperature=1.2, top_k=20, seed=3),
             SamplingParams(temperature=0.9, top_p=0.9, repetition_penalty=1.3, seed=3)]
    mixed = model.generate(prompts, max_new_tokens=8, sampling=kinds).tokens
    for i, kind in enumerate(kinds):
        alike = model.generate(prompts, max_new_tokens=8, sampling=[kind] * 4).tokens
        assert mixed[i] == alike[i], f"request {i}"
    assert mixed[0] == model.generate(prompts, max_new_tokens=8).tokens[0]
