"""The library's host sampler against the reference's frozen vectors
(/root/reference/crates/nnis-model/src/sampling.rs:290-362) and against the
tests' plain sampler."""

import numpy as np
import pytest

import plain_llama as P
from nnis_amd.errors import InvalidInput
from nnis_amd.sampling import HostSampler, SamplingParams, SplitMix64, greedy_token


def test_frozen_vectors():
    sampler = HostSampler(SamplingParams(seed=42), 4)
    assert [sampler.sample(np.zeros(4, np.float32)) for _ in range(10)] == [2, 0, 1, 1, 0, 3, 0, 3, 1, 2]
    assert HostSampler(SamplingParams(seed=7, top_k=1), 4).sample([1.0, 4.0, 4.0, -2.0]) == 1
    assert greedy_token(np.array([1.0, 4.0, 4.0, -2.0])) == 1
    nucleus = HostSampler(SamplingParams(seed=9, top_p=0.1), 3)
    assert all(nucleus.sample([3.0, 2.0, 1.0]) == 0 for _ in range(32))
    top2 = HostSampler(SamplingParams(seed=123, top_k=2), 4)
    assert all(top2.sample([4.0, 3.0, 2.0, 1.0]) <= 1 for _ in range(64))


def test_rejections():
    for bad in (dict(temperature=0.0), dict(temperature=float("nan")), dict(top_k=0), dict(top_k=5), dict(top_p=0.0),
                dict(top_p=1.1), dict(top_p=float("inf"))):
        with pytest.raises(InvalidInput):
            SamplingParams(seed=1, **bad).validate(4)
    SamplingParams(seed=1).validate(4)
    with pytest.raises(InvalidInput):
        SamplingParams(seed=1).validate(0)
    with pytest.raises(InvalidInput):
        SamplingParams(seed=-1).validate(4)
    sampler = HostSampler(SamplingParams(seed=1), 2)
    for logits in ([1.0], [1.0, float("nan")], [1.0, float("inf")]):
        with pytest.raises(InvalidInput):
            sampler.sample(logits)


def test_generator_matches_the_plain_one():
    ours, plain = SplitMix64(2**64 - 5), P.PlainSplitMix64(2**64 - 5)
    assert [ours.next_u64() for _ in range(50)] == [plain.next_u64() for _ in range(50)]
    assert 0.0 <= ours.next_unit() < 1.0


@pytest.mark.parametrize("options", [dict(), dict(temperature=0.8), dict(top_k=7), dict(top_p=0.6),
                                     dict(temperature=1.7, top_k=20, top_p=0.9)])
def test_matches_the_plain_sampler(options):
    rng = np.random.default_rng(5)
    logits = (rng.standard_normal(300) * 3).astype(np.float32)
    logits[17] = logits[230]  # a tie
    ours = HostSampler(SamplingParams(seed=77, **options), 300)
    plain = P.PlainSplitMix64(77)
    for _ in range(200):
        assert ours.sample(logits) == P.plain_sample(logits, plain, **{"temperature": 1.0, **options})
