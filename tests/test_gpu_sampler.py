"""GPU parity of the stochastic sampler modules through the C ABI, shaped like the
reference's SoftmaxLogitsTests / SortTests / CumulativeSumTests /
SampleTopPTests, plus the sizes and edge cases those leave out.

Bars: sort, sample_top_p and every token id are bit-exact against the oracle;
cumulative_sum is bit-exact in the reference's integer regime and within one
fp16 step of the fp64 prefix sums otherwise; softmax_logits is within one fp16
step of the reference's sequential fp32 restatement and within 2e-3 of the
fp64 oracle (indices bit-exact).
"""
import numpy as np
import pytest

from managedllama2_amd import capi, synth
from gpu_util import ulp_diff, up

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 7, 8, 125, 999, 1000, 32000, 32768, 32769, 50001, 65536]


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16)


def SoftmaxLogits(x, temperature):
    d, idx = up(x), up(np.full(x.size, -1, np.int32))
    capi.call("llama2_softmax_logits", d.ptr, x.size, temperature, idx.ptr)
    return d.to_host(), idx.to_host()


def Sort(keys, values):
    k, v = up(keys), up(values)
    capi.call("llama2_sort", k.ptr, v.ptr, keys.size)
    return k.to_host(), v.to_host()


def CumulativeSum(x):
    d = up(x)
    capi.call("llama2_cumulative_sum", d.ptr, x.size)
    return d.to_host()


def SampleTopP(x, indices, threshold, pos=0):
    d, i, r = up(x), up(indices), up(np.full(pos + 2, -7, np.int32))
    capi.call("llama2_sample_top_p", d.ptr, i.ptr, x.size, threshold, r.ptr, pos)
    out = r.to_host()
    assert out[pos + 1] == -7 and (pos == 0 or out[pos - 1] == -7)
    return int(out[pos])


class TestSoftmaxLogits:
    def test_reference_regime(self, oracle):
        # Test_SoftmaxLogits (test/SoftmaxLogitsTests.cs:75-94): 16 uniform values, temperature 1
        rng = synth.rng_for(901)
        for _ in range(10):
            x = f16(rng.random(16))
            got, idx = SoftmaxLogits(x, 1.0)
            want, widx = oracle.ref_softmax_logits(x, 1.0)
            assert np.array_equal(idx, widx)
            assert ulp_diff(got, want).max() <= 1

    @pytest.mark.parametrize("size", SIZES)
    @pytest.mark.parametrize("temperature", [0.5, 1.0, 1.7])
    def test_vs_oracle(self, oracle, size, temperature):
        rng = synth.rng_for(902, size)
        x = synth.normal_f16(rng, size, 2.0)
        got, idx = SoftmaxLogits(x, temperature)
        assert np.array_equal(idx, np.arange(size, dtype=np.int32))
        want, _ = oracle.ref_softmax_logits(x, temperature)
        assert ulp_diff(got, want).max() <= 1
        assert np.mean(got.view(np.uint16) == want.view(np.uint16)) >= 0.97
        exact = oracle.f64_softmax_logits(x, temperature)
        # 2e-3 relative, plus one step of the fp16 subnormal grid the small probabilities are stored on
        assert np.all(np.abs(got.astype(np.float64) - exact) <= 2e-3 * exact + 2.0 ** -24)

    def test_peaked_and_flat(self, oracle):
        x = f16(np.zeros(32000))
        got, _ = SoftmaxLogits(x, 0.3)
        assert np.all(got == np.float16(1.0 / 32000))
        x[12345] = 30.0
        got, _ = SoftmaxLogits(x, 0.5)  # exp(-60) underflows: a one-hot row
        assert got[12345] == 1.0 and np.count_nonzero(got) == 1

    def test_rejects(self):
        d, idx = up(f16(np.zeros(8))), up(np.zeros(8, np.int32))
        assert capi.raw("llama2_softmax_logits", d.ptr, 8, 0.0, idx.ptr) == capi.ERR_INVALID_ARGUMENT
        assert capi.raw("llama2_softmax_logits", d.ptr, 0, 1.0, idx.ptr) == capi.ERR_INVALID_ARGUMENT
        assert capi.raw("llama2_softmax_logits", d.ptr, capi.MAX_SAMPLER_SIZE + 1, 1.0, idx.ptr) == capi.ERR_UNSUPPORTED
        assert capi.raw("llama2_softmax_logits", None, 8, 1.0, idx.ptr) == capi.ERR_INVALID_ARGUMENT


class TestSort:
    def test_reference_regime(self, oracle):
        # Test_Sort (test/SortTests.cs:57-90): 32000 integers in [0, 1024) as fp16, indices 0..n-1.
        # The reference checks the keys only (its CPU sort is unstable); the stable order is checked here.
        rng = synth.rng_for(911)
        keys = rng.integers(0, 1024, 32000).astype(np.float16)
        vals = np.arange(32000, dtype=np.int32)
        k, v = Sort(keys, vals)
        wk, wv = oracle.ref_sort(keys, vals)
        assert np.array_equal(k.view(np.uint16), wk.view(np.uint16))
        assert np.array_equal(v, wv)

    @pytest.mark.parametrize("size", SIZES)
    def test_sizes(self, oracle, size):
        rng = synth.rng_for(912, size)
        keys = synth.normal_f16(rng, size, 3.0)
        keys[rng.integers(0, size, max(1, size // 10))] = keys[0]  # ties
        vals = rng.integers(-2 ** 31, 2 ** 31 - 1, size).astype(np.int32)
        k, v = Sort(keys, vals)
        wk, wv = oracle.ref_sort(keys, vals)
        assert np.array_equal(k.view(np.uint16), wk.view(np.uint16))
        assert np.array_equal(v, wv)

    def test_probabilities_after_softmax(self, oracle):
        rng = synth.rng_for(913)
        p, idx = oracle.ref_softmax_logits(synth.normal_f16(rng, 32000, 2.0), 0.5)
        k, v = Sort(p, idx)
        wk, wv = oracle.ref_sort(p, idx)
        assert np.array_equal(k.view(np.uint16), wk.view(np.uint16)) and np.array_equal(v, wv)
        assert np.all(k[:-1] >= k[1:])

    def test_special_values_and_repeats(self, oracle):
        bits = np.array([0x0000, 0x8000, 0x7C00, 0xFC00, 0x3C00, 0x8001, 0x0001, 0x7BFF, 0xFBFF] * 50, np.uint16)
        keys = bits.view(np.float16)
        vals = np.arange(keys.size, dtype=np.int32)
        k, v = Sort(keys, vals)
        wk, wv = oracle.ref_sort(keys, vals)
        assert np.array_equal(k.view(np.uint16), wk.view(np.uint16)) and np.array_equal(v, wv)
        # sorting twice changes nothing (idempotent), and repeated calls reuse the library's second buffer
        k2, v2 = Sort(k, v)
        assert np.array_equal(k2.view(np.uint16), k.view(np.uint16)) and np.array_equal(v2, v)

    def test_rejects(self):
        k, v = up(f16(np.zeros(8))), up(np.zeros(8, np.int32))
        assert capi.raw("llama2_sort", k.ptr, v.ptr, 0) == capi.ERR_INVALID_ARGUMENT
        assert capi.raw("llama2_sort", k.ptr, v.ptr, capi.MAX_SAMPLER_SIZE + 1) == capi.ERR_UNSUPPORTED
        assert capi.raw("llama2_sort", k.ptr, None, 8) == capi.ERR_INVALID_ARGUMENT


class TestCumulativeSum:
    def test_reference_regime(self, oracle):
        # Test_CumulativeSum (test/CumulativeSumTests.cs:51-68): 32000 integers in [-1000, 1000], ten vectors
        rng = synth.rng_for(921)
        for _ in range(10):
            x = rng.integers(-1000, 1001, 32000).astype(np.float16)
            got = CumulativeSum(x)
            want = oracle.ref_cumulative_sum(x)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16))

    @pytest.mark.parametrize("size", SIZES)
    def test_probabilities(self, oracle, size):
        rng = synth.rng_for(922, size)
        p, _ = oracle.ref_softmax_logits(synth.normal_f16(rng, size, 2.0), 1.0)
        got = CumulativeSum(p)
        exact = oracle.f64_cumulative_sum(p)
        assert ulp_diff(got, oracle.round_d2h(exact)).max() <= 1
        assert np.all(np.diff(got.astype(np.float32)) >= 0)
        want = oracle.ref_cumulative_sum(p)
        assert ulp_diff(got, want).max() <= 1

    def test_rejects(self):
        d = up(f16(np.zeros(8)))
        assert capi.raw("llama2_cumulative_sum", d.ptr, -1) == capi.ERR_INVALID_ARGUMENT
        assert capi.raw("llama2_cumulative_sum", None, 8) == capi.ERR_INVALID_ARGUMENT


class TestSampleTopP:
    def test_reference_regime(self, oracle):
        # Test_SampleTopP (test/SampleTopPTests.cs:48-65): 16 uniform values, 16 random indices, threshold 0.9
        rng = synth.rng_for(931)
        for _ in range(10):
            x = f16(rng.random(16))
            idx = rng.integers(0, 16, 16).astype(np.int32)
            assert SampleTopP(x, idx, 0.9) == oracle.ref_sample_top_p(x, idx, 0.9)

    @pytest.mark.parametrize("size", SIZES)
    def test_cdf(self, oracle, size):
        rng = synth.rng_for(932, size)
        p, _ = oracle.ref_softmax_logits(synth.normal_f16(rng, size, 2.0), 1.0)
        cdf = oracle.ref_cumulative_sum(p)
        idx = rng.permutation(size).astype(np.int32)
        for thr in [0.0, 1e-4, 0.25, 0.5, 0.9, 0.999, 1.0, 1.5, float(cdf[size // 2])]:
            assert SampleTopP(cdf, idx, thr, pos=3) == oracle.ref_sample_top_p(cdf, idx, thr)

    def test_unsorted_values_take_the_first_hit(self, oracle):
        x = f16(np.zeros(40000))
        x[[39999, 17, 20000]] = 1.0
        idx = np.arange(40000, dtype=np.int32)[::-1].copy()
        assert SampleTopP(x, idx, 0.5) == idx[17] == oracle.ref_sample_top_p(x, idx, 0.5)


def fused_sample(logits, temperature, top_p, coin, pos=1):
    d, idx, r = up(logits), up(np.zeros(logits.size, np.int32)), up(np.full(pos + 1, -7, np.int32))
    capi.call("llama2_sample", d.ptr, idx.ptr, logits.size, temperature, top_p, coin, r.ptr, pos)
    return int(r.to_host()[pos]), d.to_host(), idx.to_host()


def module_sample(logits, temperature, top_p, coin, pos=1):
    d, idx, r = up(logits), up(np.zeros(logits.size, np.int32)), up(np.full(pos + 1, -7, np.int32))
    n = logits.size
    capi.call("llama2_softmax_logits", d.ptr, n, temperature, idx.ptr)
    threshold = np.float32(coin)
    if 0 < top_p < 1:
        capi.call("llama2_sort", d.ptr, idx.ptr, n)
        threshold = np.float32(coin) * np.float32(top_p)
    capi.call("llama2_cumulative_sum", d.ptr, n)
    capi.call("llama2_sample_top_p", d.ptr, idx.ptr, n, float(threshold), r.ptr, pos)
    return int(r.to_host()[pos]), d.to_host(), idx.to_host()


class TestSample:
    @pytest.mark.parametrize("size", [5, 1000, 32000, 40000])
    @pytest.mark.parametrize("top_p", [0.9, 1.0, 0.0, 0.3])
    def test_one_launch_equals_the_four_modules(self, oracle, size, top_p):
        rng = synth.rng_for(941, size)
        logits = synth.normal_f16(rng, size, 2.0)
        for coin in (0.0, 0.37, 0.93, 0.999999):
            t1, cdf1, idx1 = fused_sample(logits, 0.7, top_p, coin)
            t2, cdf2, idx2 = module_sample(logits, 0.7, top_p, coin)
            assert t1 == t2
            assert np.array_equal(cdf1.view(np.uint16), cdf2.view(np.uint16)) and np.array_equal(idx1, idx2)
            # the token is the oracle's pick on the GPU's own cdf (integer step: exact) ...
            thr = np.float32(coin) * np.float32(top_p) if 0 < top_p < 1 else np.float32(coin)
            assert t1 == oracle.ref_sample_top_p(cdf1, idx1, float(thr))
            # ... and the cdf is the oracle's up to one fp16 step per stage
            work = logits.copy()
            p, widx = oracle.ref_softmax_logits(work, 0.7)
            if 0 < top_p < 1:
                p, widx = oracle.ref_sort(p, widx)
            wcdf = oracle.ref_cumulative_sum(p)
            assert np.max(np.abs(cdf1.astype(np.float64) - wcdf.astype(np.float64))) <= 2.0 ** -9

    def test_tokens_match_the_oracle_on_a_small_vocabulary(self, oracle):
        logits = f16([1.0, 3.0, 2.0, -1.0, 0.5, 2.5, -3.0, 0.0])
        n = 400
        for top_p in (0.8, 1.0):
            agree = 0
            for i in range(n):
                coin = (i + 0.5) / n
                tok, _, _ = fused_sample(logits, 0.8, top_p, coin)
                agree += tok == oracle.ref_sample(logits, 0.8, top_p, coin)
            assert agree >= n - 2  # a coin within one fp16 step of a cdf boundary may fall either way

    def test_distribution(self, oracle):
        logits = f16([1.0, 3.0, 2.0, -1.0])
        T, n = 0.8, 1000
        p = np.exp(logits.astype(np.float64) / T)
        p /= p.sum()
        counts = np.zeros(4)
        for i in range(n):
            counts[fused_sample(logits, T, 1.0, (i + 0.5) / n)[0]] += 1
        assert np.max(np.abs(counts / n - p)) < 5e-3
