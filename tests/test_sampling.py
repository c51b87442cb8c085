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


def test_rows_drawn_together_give_what_each_gives_alone():
    """The draw for many rows at once against the draw for one: the same tokens, and each stream advanced by one
    number, for candidates with equal values, every cut of top_k and top_p, and one to a thousand candidates."""
    import numpy as np

    from rvllm_amd.sampling.sampler import sample_rows

    gen = np.random.default_rng(3)
    for k in (1, 2, 7, 50, 1024):
        rows = 40
        vals = (gen.standard_normal((rows, k)) * 3).astype(np.float32)
        vals[::3] = np.round(vals[::3])  # many equal values: the lower id goes first
        ids = np.stack([gen.permutation(5000)[:k] for _ in range(rows)]).astype(np.int32)
        top_k = [int(gen.integers(0, k + 1)) for _ in range(rows)]
        top_p = [float(x) for x in gen.choice([0.0, 0.1, 0.5, 0.9, 0.999, 1.0], size=rows)]
        for seed in range(3):
            together = sample_rows(vals, ids, top_k, top_p, [SplitMix64(seed * 100 + r) for r in range(rows)], 5000)
            streams = [SplitMix64(seed * 100 + r) for r in range(rows)]
            alone = [sample_from_candidates(list(zip(vals[r].tolist(), ids[r].tolist())), top_k[r], top_p[r], streams[r],
                                            5000) for r in range(rows)]
            assert together == alone, (k, seed)
    # each stream moves by exactly one number
    a, b = SplitMix64(9), SplitMix64(9)
    sample_rows(np.array([[0.5, 1.5]], dtype=np.float32), np.array([[3, 4]], dtype=np.int32), [0], [1.0], [a])
    b.next_f64()
    assert a.next_u64() == b.next_u64()


def test_rows_drawn_together_refuse_what_one_row_refuses():
    import numpy as np

    from rvllm_amd.sampling.sampler import sample_rows

    one = lambda v, i, tk=0, tp=1.0, vocab=None: sample_rows(np.array([v], dtype=np.float32), np.array([i], dtype=np.int32),
                                                           [tk], [tp], [SplitMix64(1)], vocab)
    for v in ([1.0, math.nan], [math.inf, 0.0]):
        with pytest.raises(SamplingError, match="finite"):
            one(v, [1, 2])
    with pytest.raises(SamplingError, match="top_k"):
        one([1.0], [1], tk=2)
    with pytest.raises(SamplingError, match="top_p"):
        one([1.0], [1], tp=math.nan)
    with pytest.raises(SamplingError, match="below vocab"):
        one([1.0], [8], vocab=8)
    assert one([1.0], [7], vocab=8) == [7]


def test_when_the_device_can_draw_for_a_step():
    """Steps follow one another for requests that sample, whatever numbers of candidates they ask for (the device
    selects as many as the one that asks for most; each keeps its own); greedy requests among them keep one."""
    from rvllm_amd.sampling.sampler import DeviceDraws

    greedy, a, b = SamplingParams(), SamplingParams(0.8, 20, 0.9, seed=1), SamplingParams(1.2, 20, 1.0, seed=2)
    assert DeviceDraws.usable(1000, [a, b, greedy])
    assert DeviceDraws.usable(1000, [a, SamplingParams(0.8, 50, 1.0)])
    assert not DeviceDraws.usable(1000, [greedy, greedy])  # nothing to draw: the arg-max does it
    assert DeviceDraws.usable(300, [SamplingParams(0.8, 0, 1.0), greedy])  # the whole of a small vocabulary
    assert not DeviceDraws.usable(5000, [SamplingParams(0.8, 0, 1.0)])  # refused for a large one, as on the host
