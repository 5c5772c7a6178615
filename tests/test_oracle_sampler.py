"""Pins the CPU oracle's restatement of the stochastic sampler
(src/Sampler.cs:48-67; kernels softmax_logits, sort, cumulative_sum,
sample_top_p) against what the mathematics fixes and against the regimes the
reference's own tests use (test/SoftmaxLogitsTests.cs, SortTests.cs,
CumulativeSumTests.cs, SampleTopPTests.cs)."""
import math

import numpy as np

from managedllama2_amd import synth


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16)


def test_softmax_logits_two_point_logistic(oracle):
    # softmax([a, b] / T) = (sigma(d), 1 - sigma(d)) with d = (a - b) / T
    for a, b, T in [(2.0, 0.0, 2.0), (0.0, 0.0, 0.7), (-1.5, 3.0, 0.5), (4.0, 1.0, 1.0)]:
        p, idx = oracle.ref_softmax_logits(f16([a, b]), T)
        d = (a - b) / T
        want = 1.0 / (1.0 + math.exp(-d))
        assert abs(float(p[0]) - want) < 1.5e-3 and abs(float(p[1]) - (1 - want)) < 1.5e-3
        assert list(idx) == [0, 1]


def test_softmax_logits_is_softmax_of_scaled_logits(oracle):
    rng = synth.rng_for(801)
    x = synth.normal_f16(rng, 32000, 2.0)
    for T in (1.0, 0.5, 1.7):
        p, idx = oracle.ref_softmax_logits(x, T)
        assert np.array_equal(idx, np.arange(32000, dtype=np.int32))
        scaled = (x.astype(np.float32) / np.float32(T)).astype(np.float16)
        q = oracle.ref_softmax(scaled)  # pinned separately (test_oracle_ops.py)
        # ref_softmax normalises the unrounded exponentials, softmax_logits the fp16-rounded ones
        assert np.max(np.abs(p.astype(np.float64) - q.astype(np.float64))) <= 2 ** -11 * float(q.max()) + 1e-7
        assert abs(float(p.astype(np.float64).sum()) - 1.0) < 2e-3
        exact = oracle.f64_softmax_logits(x, T)
        big = exact > 1e-4
        assert np.max(np.abs(p.astype(np.float64)[big] / exact[big] - 1)) < 1.5e-3
    # a higher temperature flattens the distribution
    assert oracle.ref_softmax_logits(x, 2.0)[0].max() < oracle.ref_softmax_logits(x, 0.5)[0].max()


def test_sort_is_the_stable_descending_sort(oracle):
    rng = synth.rng_for(802)
    # the reference's regime: 32000 integers in [0, 1024) as fp16 (test/SortTests.cs:57-63): many ties
    keys = rng.integers(0, 1024, 32000).astype(np.float16)
    vals = np.arange(32000, dtype=np.int32)
    k, v = oracle.ref_sort(keys, vals)
    order = np.argsort(-keys.astype(np.float32), kind="stable")
    assert np.array_equal(k, keys[order]) and np.array_equal(v, vals[order])
    # python's sorted (stable) on a small ragged input with negative keys
    keys = f16([0.5, -2.0, 7.0, 0.5, 0.25, 7.0, -2.0, 1e-7, 65504.0, 0.5, -65504.0])
    vals = np.array([10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20], np.int32)
    k, v = oracle.ref_sort(keys, vals)
    want = sorted(zip(keys.tolist(), vals.tolist()), key=lambda kv: -kv[0])
    assert [float(a) for a in k] == [a for a, _ in want] and list(v) == [b for _, b in want]
    # probabilities: any permutation of the values is carried with its key
    p = oracle.ref_softmax_logits(synth.normal_f16(rng, 999, 3.0), 1.0)[0]
    perm = rng.permutation(999).astype(np.int32)
    k, v = oracle.ref_sort(p, perm)
    assert np.all(k[:-1] >= k[1:])
    lookup = {int(t): float(pp) for t, pp in zip(perm, p)}
    assert all(lookup[int(t)] == float(kk) for t, kk in zip(v, k))
    assert sorted(v.tolist()) == list(range(999))


def test_sort_total_order_on_special_values(oracle):
    keys = np.array([0x0000, 0x8000, 0x7C00, 0xFC00, 0x3C00, 0x8001, 0x0001], np.uint16).view(np.float16)
    k, v = oracle.ref_sort(keys, np.arange(7, dtype=np.int32))
    # +inf, 1, smallest subnormal, +0, -0, -smallest subnormal, -inf
    assert list(v) == [2, 4, 6, 0, 1, 5, 3]


def test_cumulative_sum_integer_regime_and_fp64(oracle):
    rng = synth.rng_for(803)
    # the reference's regime (test/CumulativeSumTests.cs:51-57): integers in [-1000, 1000], exact in fp32
    ints = rng.integers(-1000, 1001, 32000)
    got = oracle.ref_cumulative_sum(ints.astype(np.float16))
    with np.errstate(over="ignore"):  # the random walk leaves the fp16 range: both sides give inf
        want = np.cumsum(ints.astype(np.int64)).astype(np.float64).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # probabilities: fp32 running sum against the fp64 one
    p = oracle.ref_softmax_logits(synth.normal_f16(rng, 32000, 2.0), 1.0)[0]
    got = oracle.ref_cumulative_sum(p).astype(np.float64)
    exact = oracle.f64_cumulative_sum(p)
    assert np.array_equal(exact, np.cumsum(p.astype(np.float64)))
    assert np.max(np.abs(got - exact)) <= 2 ** -11 * 1.001  # one fp16 rounding of a value <= 1
    assert np.all(np.diff(got) >= 0)


def test_sample_top_p_brute_force(oracle):
    rng = synth.rng_for(804)
    for _ in range(20):
        x = rng.random(16).astype(np.float16)  # the reference's regime: 16 uniform values, unsorted
        idx = rng.integers(0, 16, 16).astype(np.int32)
        for thr in [0.0, 0.1, 0.5, 0.9, 0.999, 1.5] + [float(t) for t in x[:4]]:
            hits = [i for i in range(16) if float(x[i]) >= np.float32(thr)]
            want = idx[hits[0]] if hits and hits[0] < 15 else idx[15]
            assert oracle.ref_sample_top_p(x, idx, thr) == want


def test_sample_distribution_and_branches(oracle):
    logits = f16([1.0, 3.0, 2.0, -1.0])
    # temperature 0 and prompt positions: src/Sampler.cs:44-47
    assert oracle.ref_sample(logits, 0.0, 0.9, 0.3) == 1
    assert oracle.ref_sample(logits, 0.8, 0.9, 0.3, generate_token=False) == -1
    # top_p outside (0, 1): plain inverse-CDF sampling in index order (src/Sampler.cs:52-55)
    T, n = 0.8, 4000
    p = np.exp(logits.astype(np.float64) / T)
    p /= p.sum()
    counts = np.zeros(4)
    for i in range(n):
        counts[oracle.ref_sample(logits, T, 1.0, (i + 0.5) / n)] += 1
    assert np.max(np.abs(counts / n - p)) < 3e-3
    # 0 < top_p < 1: sorted by probability, threshold coin * top_p (src/Sampler.cs:57-61):
    # the nucleus is the shortest sorted prefix whose mass reaches top_p
    top_p = 0.8
    order = np.argsort(-p)
    counts = np.zeros(4)
    for i in range(n):
        counts[oracle.ref_sample(logits, T, top_p, (i + 0.5) / n)] += 1
    cdf = np.cumsum(p[order])
    nucleus = order[:int(np.searchsorted(cdf, top_p)) + 1]
    assert set(np.nonzero(counts)[0]) == set(nucleus.tolist())
    want = np.diff(np.concatenate([[0.0], np.minimum(cdf, top_p)])) / top_p
    assert np.max(np.abs(counts[order] / n - want)) < 4e-3


def test_coin_known_answer_and_range(oracle):
    # splitmix64, seed 0, first output 0xE220A8397B1DCDAF: its top 24 bits / 2^24
    assert oracle.coin(0, 0) == 0xE220A8 / 2.0 ** 24
    # second output of the same stream: 0x6E789E6AA1B965F4
    assert oracle.coin(0, 1) == 0x6E789E / 2.0 ** 24
    c = np.array([oracle.coin(1234, i) for i in range(4000)])
    assert c.min() >= 0.0 and c.max() < 1.0 and abs(c.mean() - 0.5) < 0.02
    assert len(set(c.tolist())) > 3990
