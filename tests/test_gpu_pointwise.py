"""GPU parity of RMSNorm, RoPE, softmax, argmax and embedding through the C
ABI, shaped like the reference's RMSNormTests / RoPETests / SoftmaxTests /
ArgmaxTests / EmbeddingTableTests."""
import numpy as np
import pytest

from managedllama2_amd import capi, synth
from gpu_util import assert_close, ulp_diff, up

pytestmark = pytest.mark.gpu


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16)


class TestRMSNorm:
    def RMSNorm(self, v1, v2, in_place=False):
        a, g = up(v1), up(v2)
        out = a if in_place else up(np.zeros(v1.size, np.float16))
        capi.call("llama2_rmsnorm", out.ptr, a.ptr, g.ptr, v1.size, 1e-5)
        return out.to_host()

    @pytest.mark.parametrize("v,g", [([1, 2, 3], [4, 5, 6]), ([6, 2, 6], [1, 9, 7])])
    def test_inline_vectors_exact(self, oracle, v, g):
        # Test_RMSNorm (test/RMSNormTests.cs:63-75)
        expected = oracle.ref_rmsnorm(f16(v), f16(g))
        assert np.array_equal(self.RMSNorm(f16(v), f16(g)).view(np.uint16), expected.view(np.uint16))

    @pytest.mark.parametrize("n", [4096, 5120, 1, 1000, 9999])
    def test_vs_fp64_and_in_place(self, oracle, n):
        rng = synth.rng_for(301, n)
        x = synth.normal_f16(rng, n, 3.0)
        g = f16(1 + 0.2 * rng.standard_normal(n))
        want = oracle.f64_rmsnorm(x, g)
        out = self.RMSNorm(x, g)
        assert_close(out, want, "rmsnorm %d" % n)
        assert ulp_diff(out, oracle.ref_rmsnorm(x, g, square_in_half=False)).max() <= 1
        assert np.array_equal(self.RMSNorm(x, g, in_place=True).view(np.uint16), out.view(np.uint16))


class TestRoPE:
    def RoPE(self, q, k, dim, seq_len, n_heads, n_kv_heads, pos, theta=10000.0):
        sq, sk = up(q), up(k)
        kv_dim = dim * n_kv_heads // n_heads
        head_size = dim // n_heads
        offset = pos * kv_dim
        capi.call("llama2_rope", sq.ptr, sk.offset_pointer(offset), n_kv_heads, head_size, pos, theta, n_heads)
        return sq.to_host(), sk.to_host()

    def test_reference_geometry(self, oracle):
        # Test_RoPE (test/RoPETests.cs:94-118): dim 128, 32 heads (head_size 4), seq 20, pos 0..18
        rng = synth.rng_for(311)
        seq_len, dim, heads = 20, 128, 32
        q, k = f16(rng.random(dim)), f16(rng.random(dim * seq_len))
        for pos in range(seq_len - 1):
            aq, ak = self.RoPE(q, k, dim, seq_len, heads, heads, pos)
            eq, ekrow = oracle.ref_rope(q, k[pos * dim:(pos + 1) * dim], dim, heads, heads, pos)
            ek = k.copy()
            ek[pos * dim:(pos + 1) * dim] = ekrow
            assert ulp_diff(aq, eq).max() <= 1, pos
            assert ulp_diff(ak, ek).max() <= 1, pos
            untouched = np.ones(k.size, bool)
            untouched[pos * dim:(pos + 1) * dim] = False
            assert np.array_equal(ak[untouched], k[untouched])

    @pytest.mark.parametrize("heads,hs,pos", [(32, 128, 0), (32, 128, 1), (32, 128, 4095), (40, 128, 777)])
    def test_llama_geometry_vs_fp64(self, oracle, heads, hs, pos):
        rng = synth.rng_for(312, heads, pos)
        dim = heads * hs
        q, krow = synth.normal_f16(rng, dim), synth.normal_f16(rng, dim)
        sq, sk = up(q), up(krow)
        capi.call("llama2_rope", sq.ptr, sk.ptr, heads, hs, pos, 10000.0, heads)
        wq, wk = oracle.f64_rope(q, krow, heads, heads, hs, pos)
        # The reference computes the angle pos*freq in fp32 (native/rope_kernel.cu:8-12),
        # so the angle itself is off by up to ~pos*2^-22 rad; the rotated pair moves by
        # that angle error times the pair's norm, plus the fp16 rounding of the result.
        for got, want, src in ((sq.to_host(), wq, q), (sk.to_host(), wk, krow)):
            v = src.astype(np.float64).reshape(heads, 2, hs // 2)
            pair_norm = np.sqrt(v[:, 0] ** 2 + v[:, 1] ** 2)
            bound = np.repeat(pair_norm[:, None, :], 2, axis=1).reshape(-1) * (pos * 2.0 ** -21 + 2.0 ** -10) + 1e-7
            assert np.all(np.abs(got.astype(np.float64) - want) <= bound)
        # and it tracks the fp32 restatement of the reference's CPU check closely
        rq, rk = oracle.ref_rope(q, krow, dim, heads, heads, pos)
        assert np.max(np.abs(sq.to_host().astype(np.float64) - rq.astype(np.float64))) <= 4 * (pos * 2.0 ** -21 + 2.0 ** -10)
        if pos == 0:
            assert np.array_equal(sq.to_host(), q) and np.array_equal(sk.to_host(), krow)

    def test_fewer_kv_heads(self, oracle):
        rng = synth.rng_for(313)
        heads, kvh, hs, pos = 8, 2, 64, 5
        q, krow = synth.normal_f16(rng, heads * hs), synth.normal_f16(rng, heads * hs)
        sq, sk = up(q), up(krow)
        capi.call("llama2_rope", sq.ptr, sk.ptr, kvh, hs, pos, 10000.0, heads)
        wq, wk = oracle.f64_rope(q, krow, heads, kvh, hs, pos)
        assert_close(sq.to_host(), wq, "rope q")
        k_out = sk.to_host()
        assert_close(k_out[: kvh * hs], wk[: kvh * hs], "rope k")
        assert np.array_equal(k_out[kvh * hs:], krow[kvh * hs:])


class TestSoftmax:
    def Softmax(self, x, n_rows=1):
        x1 = up(x)
        capi.call("llama2_softmax", x1.ptr, x.size // n_rows, n_rows)
        return x1.to_host()

    def test_reference_vectors(self, oracle):
        # Test_Softmax (test/SoftmaxTests.cs:61-78): 10 vectors of 16 uniform values
        rng = synth.rng_for(321)
        for _ in range(10):
            x = f16(rng.random(16))
            assert ulp_diff(self.Softmax(x), oracle.ref_softmax(x)).max() <= 1

    @pytest.mark.parametrize("size,rows", [(512, 32), (2048, 32), (4096, 32), (8192, 3), (1, 5), (1025, 7)])
    def test_vs_fp64(self, oracle, size, rows):
        rng = synth.rng_for(322, size)
        x = synth.normal_f16(rng, size * rows, 2.0)
        got = self.Softmax(x, rows)
        want = oracle.f64_softmax(x, size, rows)
        for r in range(rows):
            assert_close(got[r * size:(r + 1) * size], want[r * size:(r + 1) * size], "softmax row %d" % r)
        assert np.allclose(got.astype(np.float64).reshape(rows, size).sum(1), 1, atol=2e-2)

    def test_all_negative_short_row(self, oracle):
        # the reference kernel seeds idle threads' maximum with 0; the result is still the softmax
        x = f16([-9.0, -7.5, -8.25])
        assert_close(self.Softmax(x), oracle.f64_softmax(x, 3, 1), "negative row")

    def test_too_long(self):
        x = up(np.zeros(16, np.float16))
        assert capi.raw("llama2_softmax", x.ptr, capi.MAX_SOFTMAX_SIZE + 1, 1) == capi.ERR_UNSUPPORTED


class TestArgmax:
    def Argmax(self, logits, n, pos=0, write=True, initial=-7):
        x = up(logits)
        result = up(np.full(pos + 1, initial, np.int32))
        capi.call("llama2_argmax", x.ptr, n, result.ptr, pos, 1 if write else 0)
        return int(result[pos])

    def test_reference_vector(self, oracle):
        # test/ArgmaxTests.cs:48-64
        rng = synth.rng_for(331)
        x = f16(rng.random(10))
        assert self.Argmax(x, 10) == oracle.ref_argmax(x)

    def test_vocab_with_ties_is_bit_exact(self, oracle):
        rng = synth.rng_for(332)
        for trial in range(5):
            x = synth.normal_f16(rng, 32000, 0.02 * 30)
            m = x.max()
            ties = rng.integers(0, 32000, 4)
            x[ties] = m
            assert self.Argmax(x, 32000) == oracle.ref_argmax(x) == int(np.argmax(x))
        x = np.full(32000, -3.0, np.float16)
        assert self.Argmax(x, 32000) == 0
        x[31999] = -2.0
        assert self.Argmax(x, 32000) == 31999

    def test_ragged_sizes_and_unaligned_input(self, oracle):
        # 16-byte loads over whole groups of 8, the remainder one by one; an input that is not
        # 16-byte aligned takes the element-wise path altogether
        rng = synth.rng_for(334)
        for n in (1, 7, 8, 9, 1023, 1024, 8191, 8195, 32003):
            x = synth.normal_f16(rng, n + 3, 1.0)
            d = up(x)
            result = up(np.full(1, -7, np.int32))
            for off in (0, 1, 3):
                want = oracle.ref_argmax(x[off:off + n])
                capi.call("llama2_argmax", d.ptr + 2 * off, n, result.ptr, 0, 1)
                assert int(result[0]) == want == int(np.argmax(x[off:off + n])), (n, off)
                x2 = x.copy()
                x2[off + n - 1] = 100.0  # the winner in the tail
                d2 = up(x2)
                capi.call("llama2_argmax", d2.ptr + 2 * off, n, result.ptr, 0, 1)
                assert int(result[0]) == n - 1, (n, off)

    def test_write_token_flag_and_position(self):
        rng = synth.rng_for(333)
        x = f16(rng.random(100))
        assert self.Argmax(x, 100, pos=3, write=False) == -7
        assert self.Argmax(x, 100, pos=3, write=True) == int(np.argmax(x))


class TestEmbeddingTable:
    def test_embed(self):
        # Test_Embed (test/EmbeddingTableTests.cs:40-50)
        rng = synth.rng_for(341)
        table = f16(rng.random(256))
        x, t, tk = up(np.zeros(256, np.float16)), up(table), up(np.array([0], np.int32))
        capi.call("llama2_embedding", x.ptr, t.ptr, 256, tk.ptr, 0)
        assert np.array_equal(x.to_host(), table)

    def test_row_select(self, oracle):
        rng = synth.rng_for(342)
        dim, vocab = 4096, 50
        table = synth.normal_f16(rng, dim * vocab)
        tokens = np.array([7, 49, 0, 13], np.int32)
        x, t, tk = up(np.zeros(dim, np.float16)), up(table), up(tokens)
        for pos in range(4):
            capi.call("llama2_embedding", x.ptr, t.ptr, dim, tk.ptr, pos)
            assert np.array_equal(x.to_host(), oracle.ref_embedding(table, dim, tokens, pos))
