"""The host sampler's law and the random generator, against the constants the reference's
sampler test holds (engine/tests/test_sampler.cu) and the plain implementation."""
import math

import numpy as np
import pytest

import plain_llama as P
from bare_cuda_4gib_amd.sampling import MT19937_64, SamplingParams, check_sampling, sample_token, seed_for

LOGITS = np.array([math.log(0.5), math.log(0.3), math.log(0.2), -1e30], dtype=np.float32)


def test_generator_is_the_standard_one():
    g = MT19937_64()                       # default seed 5489: the 10000th draw is fixed by the C++ standard
    for _ in range(9999):
        g.next_u64()
    assert g.next_u64() == 9981545732273789042
    g = MT19937_64(7)
    assert [g.next_u64() for _ in range(3)] == [13915952638675311015, 17511516338625233250, 2165911192842364878]
    g = MT19937_64(12345)                  # std::uniform_real_distribution<double>(0, 1) over std::mt19937_64(12345)
    assert [g.uniform() for _ in range(3)] == [0.35762972288842593, 0.40044261704406114, 0.68938331700276845]


@pytest.mark.parametrize("params", [
    dict(temperature=1.0), dict(temperature=0.5), dict(temperature=1.0, top_k=2),
    dict(temperature=1.0, top_p=0.7), dict(temperature=1.0, top_k=2, top_p=0.6),
    dict(temperature=0.0), dict(temperature=2.0, top_k=1),
])
def test_frequencies(params):
    # 40,000 draws within 0.015 of the expected frequencies (test_sampler.cu:15-16, 49-61)
    p = SamplingParams(seed=1, **params)
    rng = MT19937_64(seed_for(p))
    counts = np.zeros(4)
    for _ in range(40000):
        counts[sample_token(LOGITS, p, rng)] += 1
    expected = P.sample_probabilities([float(x) for x in LOGITS], params["temperature"],
                                      params.get("top_k", 0), params.get("top_p", 1.0))
    assert np.abs(counts / 40000 - np.array(expected)).max() < 0.015


def test_flat_nucleus_over_a_large_vocabulary():
    logits = np.zeros(32000, dtype=np.float32)          # test_sampler.cu: 32000-entry flat row, top_p keeps 90 %
    p = SamplingParams(temperature=1.0, top_p=0.9, seed=3)
    rng = MT19937_64(3)
    draws = [sample_token(logits, p, rng) for _ in range(200)]
    assert max(draws) < 28801 and min(draws) >= 0       # ties keep lower ids first


def test_same_seed_same_draws():
    p = SamplingParams(temperature=0.8, seed=7)
    a, b, c = MT19937_64(seed_for(p)), MT19937_64(seed_for(p)), MT19937_64(8)
    logits = np.random.default_rng(0).normal(size=100).astype(np.float32)
    da = [sample_token(logits, p, a) for _ in range(50)]
    assert da == [sample_token(logits, p, b) for _ in range(50)]
    assert da != [sample_token(logits, p, c) for _ in range(50)]
    assert seed_for(SamplingParams(seed=-1)) != seed_for(SamplingParams(seed=-1))


def test_check_sampling():
    assert check_sampling(SamplingParams()) == ""
    for bad in (dict(temperature=-1.0), dict(temperature=float("nan")), dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-1)):
        assert check_sampling(SamplingParams(**bad)) != ""
    assert SamplingParams(temperature=0.0).greedy() and SamplingParams(temperature=2.0, top_k=1).greedy()
    assert not SamplingParams(temperature=0.5).greedy()
