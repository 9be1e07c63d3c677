"""The host sampler against the reference's vectors and against the plain sampler (no GPU)."""
import numpy as np
import pytest

from plain.sampler_plain import PlainRng, PlainSampler
from rust_inference_amd.sampling import HostSampler, SamplingParams, Xorshift64Star


def test_generator_matches_the_plain_one_and_is_in_range():
    for seed in (0, 1, 7, 0x5EED, 2 ** 63 + 5):
        a, b = Xorshift64Star(seed), PlainRng(seed)
        xs = [a.next_u64() for _ in range(50)]
        assert xs == [b.next_u64() for _ in range(50)]
    g = Xorshift64Star(3)
    fs = [g.next_f32() for _ in range(2000)]
    assert all(0.0 <= f < 1.0 for f in fs) and 0.45 < np.mean(fs) < 0.55
    assert all(f == float(np.float32(f)) for f in fs)          # 24 bits: exact in float32


def test_vectors_of_the_reference():
    # src/sampling.rs:145-187
    assert HostSampler(SamplingParams()).sample([0.1, 3.0, 2.0]) == 1
    assert HostSampler(SamplingParams(repetition_penalty=2.0)).sample([0.1, 3.0, 2.0], [1]) == 2
    s = HostSampler(SamplingParams(temperature=1.0, top_k=1))
    assert all(s.sample([0.5, 0.4, 0.6, 0.1]) == 2 for _ in range(20))
    params = SamplingParams(temperature=1.0, seed=7)
    s = HostSampler(params)
    picks = [s.sample([0.0, np.log(3.0)]) for _ in range(4000)]
    assert abs(np.mean(picks) - 0.75) < 0.03
    s2 = HostSampler(params)
    assert picks == [s2.sample([0.0, np.log(3.0)]) for _ in range(4000)]
    s = HostSampler(SamplingParams(temperature=1.0, top_p=0.5))
    assert all(s.sample([3.0, 1.0, 0.5, 0.0]) == 0 for _ in range(50))


def test_ties_go_to_the_lower_index():
    assert HostSampler(SamplingParams()).sample([1.0, 3.0, 3.0]) == 1
    # of three equal candidates top-k 2 keeps the two lower ids: id 3 is never drawn
    s = HostSampler(SamplingParams(temperature=1.0, top_k=2, seed=5))
    assert {s.sample([1.0, 2.0, 2.0, 2.0]) for _ in range(200)} == {1, 2}


def test_penalty_divides_positive_and_multiplies_negative_logits_once():
    # greedy over [2, -2, 4, 0] with ids 0 and 1 seen (twice each: counted once) and 99 outside the row:
    # penalty 2 gives [1, -4, 4, 0]; penalty 8 on a seen 4 would put it below the unseen 2
    assert HostSampler(SamplingParams(repetition_penalty=2.0)).sample([2.0, -2.0, 4.0, 0.0], [0, 1, 1, 0, 99]) == 2
    assert HostSampler(SamplingParams(repetition_penalty=8.0)).sample([2.0, -2.0, 4.0, 0.0], [2, 2]) == 0
    assert HostSampler(SamplingParams(repetition_penalty=3.0)).sample([-1.0, -2.0, -1.5], [0]) == 2    # -1 * 3 = -3


@pytest.mark.parametrize("params", [
    dict(temperature=0.8, seed=1), dict(temperature=1.3, top_k=5, seed=2), dict(temperature=0.7, top_p=0.8, seed=3),
    dict(temperature=1.0, top_k=12, top_p=0.6, repetition_penalty=1.3, seed=4), dict(repetition_penalty=1.7),
])
def test_same_tokens_as_the_plain_sampler(params):
    rng = np.random.default_rng(5)
    ours, plain = HostSampler(SamplingParams(**params)), PlainSampler(**params)
    history = [3, 9, 9, 40]
    for _ in range(60):
        logits = (2.5 * rng.normal(size=97)).astype(np.float32)
        logits[10] = logits[20]                                     # a tie in the row
        a, b = ours.sample(logits, history), plain.sample(logits, history)
        assert a == b
        history.append(a)


def test_logits_that_are_not_numbers_are_ordered_like_the_reference_orders_them():
    """The candidates are sorted by a total order over every bit pattern (f32::total_cmp in the reference,
    src/sampling.rs:96-101): a row with NaNs, infinities and both zeros is sorted without a fault (the
    sanitized build runs the same code), the same way every time, and top-k 1 takes what that order puts first:
    a positive NaN, which stands above +inf."""
    rng = np.random.default_rng(8)
    row = (2.0 * rng.normal(size=4096)).astype(np.float32)
    row[::7] = np.nan
    row[5::11] = -np.nan
    row[3], row[100], row[200], row[201] = np.inf, -np.inf, 0.0, -0.0
    s = HostSampler(SamplingParams(temperature=1.0, top_k=1, seed=2))
    assert {s.sample(row) for _ in range(5)} == {0}                      # index 0: the first positive NaN
    clean = np.where(np.isnan(row), np.float32(-1e30), row)
    clean[3] = 50.0
    t = HostSampler(SamplingParams(temperature=1.0, top_k=3, seed=2))
    picks = [t.sample(clean) for _ in range(50)]
    assert set(picks) == {3}                                             # e^(x - 50) of the others rounds to nothing
