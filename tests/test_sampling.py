"""The host side of sampling, pinned by the vectors and properties of the
reference's own tests (v3/crates/rvllm-sampling/src/sampler.rs:220-377,
params.rs)."""

import math

import pytest

from rvllm_amd.sampling.params import DEFAULT_TOP_K, SamplingError, SamplingParams
from rvllm_amd.sampling.sampler import SplitMix64, sample_from_candidates


def test_splitmix64_known_outputs():
    # First outputs of SplitMix64 from state 0 (the published test vector of
    # the generator) and from 1234567.
    rng = SplitMix64(0)
    assert [rng.next_u64() for _ in range(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    rng = SplitMix64(1234567)
    assert [rng.next_u64() for _ in range(2)] == [6457827717110365317, 3203168211198807973]


def test_rng_is_deterministic_and_in_unit_interval():
    a, b = SplitMix64(42), SplitMix64(42)
    assert [a.next_u64() for _ in range(64)] == [b.next_u64() for _ in range(64)]
    assert SplitMix64(42).next_u64() != SplitMix64(43).next_u64()
    rng = SplitMix64(7)
    assert all(0.0 <= rng.next_f64() < 1.0 for _ in range(1000))
    # 53 bits: (u64 >> 11) * 2^-53
    rng = SplitMix64(0)
    assert rng.next_f64() == (0xE220A8397B1DCDAF >> 11) * 2.0 ** -53


def test_top_k_one_is_argmax():
    rng = SplitMix64(0)
    for _ in range(32):
        assert sample_from_candidates([(1.0, 10), (3.0, 20), (2.0, 30)], 1, 1.0, rng) == 20


def test_top_p_zero_keeps_argmax_only():
    rng = SplitMix64(1)
    for _ in range(32):
        assert sample_from_candidates([(0.0, 1), (0.5, 2), (-1.0, 3)], 0, 0.0, rng) == 2


def test_arrival_order_does_not_matter():
    cands = [(0.3, 7), (0.9, 4), (0.9, 11), (-0.2, 5), (0.1, 2)]
    for seed in range(256):
        a = sample_from_candidates(list(cands), 0, 0.8, SplitMix64(seed))
        b = sample_from_candidates(list(reversed(cands)), 0, 0.8, SplitMix64(seed))
        assert a == b, seed


def test_equal_values_sort_by_lower_id_first():
    # with top_k 1 and two equal maxima the lower id is the one kept
    assert sample_from_candidates([(0.9, 11), (0.9, 4)], 1, 1.0, SplitMix64(5)) == 4


def test_empirical_frequency_tracks_softmax():
    counts = [0, 0, 0]
    rng = SplitMix64(123)
    n = 60000
    for _ in range(n):
        counts[sample_from_candidates([(2.0, 0), (1.0, 1), (0.0, 2)], 0, 1.0, rng)] += 1
    for c, p in zip(counts, [0.66524096, 0.24472847, 0.09003057]):
        assert abs(c / n - p) / p < 0.03


def test_nucleus_cut_excludes_tail():
    rng = SplitMix64(9)
    for _ in range(5000):
        assert sample_from_candidates([(2.0, 0), (1.0, 1), (0.0, 2)], 0, 0.7, rng) != 2


def test_candidates_fail_closed():
    rng = SplitMix64(0)
    for bad in ([], [(math.nan, 1)]):
        with pytest.raises(SamplingError):
            sample_from_candidates(bad, 0, 1.0, rng)
    with pytest.raises(SamplingError):
        sample_from_candidates([(1.0, 1)], 2, 1.0, rng)
    with pytest.raises(SamplingError):
        sample_from_candidates([(1.0, 1)], 0, math.nan, rng)
    with pytest.raises(SamplingError):
        sample_from_candidates([(1.0, 8)], 0, 1.0, rng, vocab=8)
    assert sample_from_candidates([(1.0, 7)], 0, 1.0, rng, vocab=8) == 7


def test_params():
    assert SamplingParams.greedy().is_greedy() and SamplingParams(temperature=0.0009).is_greedy()
    assert not SamplingParams(temperature=0.001).is_greedy()
    assert SamplingParams.sampled(0.8, 0.9, 3) == SamplingParams(0.8, DEFAULT_TOP_K, 0.9, 3)
    for bad in (SamplingParams(temperature=-0.1), SamplingParams(temperature=math.inf), SamplingParams(top_p=1.5),
                SamplingParams(top_k=1025)):
        with pytest.raises(SamplingError):
            bad.validate()
    # top_k 0 = the whole vocabulary, allowed only up to 1024 (params.rs:64-78)
    assert SamplingParams(0.8, 0).kernel_k(509) == 509
    with pytest.raises(SamplingError, match="explicit top_k"):
        SamplingParams(0.8, 0).kernel_k(262208)
    assert SamplingParams(0.8, 50).kernel_k(262208) == 50
    with pytest.raises(SamplingError):
        SamplingParams(0.8, 300).kernel_k(256)
