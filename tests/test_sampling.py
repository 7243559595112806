"""Sampling on the host (no GPU): the generator, the cuts and the draw."""

import math

import numpy as np
import pytest

import plain_lfm2
from flyweight_amd.sampling import GREEDY, SamplingConfig, XorShift64Star, defaults
from host_sampling import draw_from_candidates, host_candidates


def test_defaults_and_validation():
    # tests/test_sampling_min_p.py:17-33 of the reference
    assert defaults() == {"temperature": 0.8, "top_k": 40, "top_p": 0.95, "min_p": 0.05}
    assert (GREEDY.temperature, GREEDY.top_k, GREEDY.top_p, GREEDY.min_p) == (0.0, 20, 0.95, 0.0)
    SamplingConfig(min_p=0.0), SamplingConfig(min_p=1.0)
    for bad in (dict(min_p=1.5), dict(min_p=-0.1), dict(top_p=0.0), dict(top_p=1.1), dict(temperature=-1.0),
                dict(top_k=-1), dict(temperature=float("nan"))):
        with pytest.raises(ValueError):
            SamplingConfig(**bad)


def test_xorshift64star_matches_an_independent_evaluation():
    def independent(state):
        m = (1 << 64) - 1
        state = state or 0x9E3779B97F4A7C15
        state ^= state >> 12
        state = (state ^ (state << 25)) & m
        state ^= state >> 27
        return state, ((state * 2685821657736338717 & m) >> 11) / 2.0 ** 53
    for seed in (7, 0, 2 ** 63 + 5):
        rng, state = XorShift64Star(seed), seed
        other = plain_lfm2.XorShift64Star(seed)
        for _ in range(5):
            state, expected = independent(state)
            assert rng.uniform() == expected == other.uniform()
            assert 0.0 <= expected < 1.0
    # a hand-computed first draw of seed 7: 7 ^ (7 << 25) = 234881031, then ^ >> 27 gives 234881030
    assert XorShift64Star(7).uniform() == ((234881030 * 2685821657736338717 & (2 ** 64 - 1)) >> 11) / 2.0 ** 53


def _support(config, draws=400, seed=1):
    logits = np.array([3.0, 2.0, 1.0, 0.0], dtype=np.float32)
    values, ids = host_candidates(logits, config.top_k)
    rng = XorShift64Star(seed)
    return {draw_from_candidates(values, ids, config, rng) for _ in range(draws)}


def test_min_p_keeps_a_prefix():
    # the vectors of tests/test_sampling_min_p.py:59-71 of the reference
    assert _support(SamplingConfig(temperature=1.0, top_k=0, top_p=1.0, min_p=0.0)) == {0, 1, 2, 3}
    assert _support(SamplingConfig(temperature=1.0, top_k=0, top_p=1.0, min_p=0.2)) == {0, 1}
    assert _support(SamplingConfig(temperature=1.0, top_k=0, top_p=1.0, min_p=1.0), draws=50) == {0}


def test_top_k_and_top_p_cuts():
    assert _support(SamplingConfig(temperature=1.0, top_k=2, top_p=1.0, min_p=0.0)) == {0, 1}
    # shares 0.644, 0.237, 0.087, 0.032: 0.85 is reached by the second, 0.9 by the third
    assert _support(SamplingConfig(temperature=1.0, top_k=0, top_p=0.85, min_p=0.0)) == {0, 1}
    assert _support(SamplingConfig(temperature=1.0, top_k=0, top_p=0.9, min_p=0.0)) == {0, 1, 2}
    assert _support(SamplingConfig(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0), draws=5) == {0}


def _support_of(shares, draws=600, **settings):
    logits = np.log(np.asarray(shares, dtype=np.float64)).astype(np.float32)
    config = SamplingConfig(temperature=1.0, **settings)
    values, ids = host_candidates(logits, config.top_k)
    mine, plain = XorShift64Star(5), plain_lfm2.XorShift64Star(5)
    found = set()
    for _ in range(draws):
        token = draw_from_candidates(values, ids, config, mine)
        assert token == plain_lfm2.sample(logits, 1.0, config.top_k, config.top_p, config.min_p, plain)
        found.add(token)
    return found


def test_top_p_counts_shares_of_all_candidates_and_min_p_cuts_after_it():
    """native/src/v2_runtime.cpp:29714-29728: the nucleus is found on shares of the whole candidate
    list, then min_p shortens what is left. With shares 0.4, 0.3, 0.2, 0.1, top_p 0.5 is reached by
    the second candidate (0.7) and min_p 0.6 (floor 0.24) keeps the first two: {0, 1}. Cutting by
    min_p first and taking the nucleus of what is left (0.4 / 0.7 = 0.57 >= 0.5) would keep {0}."""
    shares = [0.4, 0.3, 0.2, 0.1]
    assert _support_of(shares, top_k=0, top_p=0.5, min_p=0.6) == {0, 1}
    assert _support_of(shares, top_k=0, top_p=0.5, min_p=0.0) == {0, 1}
    assert _support_of(shares, top_k=0, top_p=1.0, min_p=0.6) == {0, 1}
    assert _support_of(shares, top_k=0, top_p=0.35, min_p=0.6) == {0}
    # the candidate list is cut to top_k before shares are formed (:29500-29566, then :29703-29710):
    # of the best two, 0.4 / 0.7 = 0.57 reaches 0.55 alone; of all four, 0.4 would not
    assert _support_of(shares, top_k=2, top_p=0.55, min_p=0.0) == {0}
    assert _support_of(shares, top_k=0, top_p=0.55, min_p=0.0) == {0, 1}


def test_candidates_order_ties_to_the_lowest_id_and_nan_last():
    logits = np.array([1.0, 5.0, float("nan"), 5.0, -2.0], dtype=np.float32)
    values, ids = host_candidates(logits, 0)
    assert ids.tolist()[:4] == [1, 3, 0, 4] and ids[-1] == 2
    assert host_candidates(logits, 2)[1].tolist() == [1, 3]


def test_draws_follow_the_distribution_and_agree_with_the_plain_sampler():
    logits = np.random.default_rng(3).normal(size=50).astype(np.float32) * 0.5
    config = SamplingConfig(temperature=0.7, top_k=10, top_p=0.9, min_p=0.02, seed=11)
    mine, plain = XorShift64Star(11), plain_lfm2.XorShift64Star(11)
    values, ids = host_candidates(logits, config.top_k)
    counts = {}
    for _ in range(3000):
        token = draw_from_candidates(values, ids, config, mine)
        assert token == plain_lfm2.sample(logits, 0.7, 10, 0.9, 0.02, plain)
        counts[token] = counts.get(token, 0) + 1
    best = int(np.argmax(logits))
    p = np.exp((values.astype(np.float64) - values[0]) / 0.7)
    kept = [i for i in range(10) if (p[:i].sum() / p.sum()) < 0.9 and p[i] >= 0.02 * p[0]]
    share = p[0] / p[kept].sum()
    assert abs(counts[best] / 3000 - share) <= 4 * math.sqrt(share * (1 - share) / 3000)
    assert len(kept) > 3 and set(counts) == {int(ids[i]) for i in kept}
