"""GPU parity of the fp16 mat-vecs (classifier GEMV, attention scores,
weighted value sum) through the C ABI, shaped like the reference's
MatVecTests / MatVecStridedTests / VecMatTests."""
import math

import numpy as np
import pytest

from managedllama2_amd import capi, synth
from gpu_util import assert_close, ulp_diff, up

pytestmark = pytest.mark.gpu


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16)


class TestMatVec:
    def MatVec(self, matrix, vector, rows, cols):
        m, v = up(matrix), up(vector)
        result = up(np.zeros(cols, np.float16))
        capi.call("llama2_mat_vec", result.ptr, v.ptr, m.ptr, rows, cols)
        return result.to_host()

    def test_reference_shape(self, oracle):
        # Test_MatVec (test/MatVecTests.cs:58-75): rows 4096, cols 64, uniform [0,1)
        rng = synth.rng_for(201)
        rows, cols = 4096, 64
        w, x = f16(rng.random(rows * cols)), f16(rng.random(rows))
        expected = oracle.ref_matvec(w, x, rows, cols)
        actual = self.MatVec(w, x, rows, cols)
        assert ulp_diff(actual, expected).max() <= 1
        assert_close(actual, oracle.f64_matvec_f16(x, w, rows, cols), "matvec 4096x64", tol=6e-4)

    @pytest.mark.parametrize("rows,cols", [(4096, 32000), (5120, 32000), (8, 3), (1032, 129)])
    def test_vs_fp64(self, oracle, rows, cols):
        rng = synth.rng_for(202, rows, cols)
        w = synth.normal_f16(rng, rows * cols, 0.02)
        x = synth.normal_f16(rng, rows)
        assert_close(self.MatVec(w, x, rows, cols), oracle.f64_matvec_f16(x, w, rows, cols), "matvec")

    def test_errors(self):
        x, m, o = up(np.zeros(16, np.float16)), up(np.zeros(64, np.float16)), up(np.zeros(4, np.float16))
        assert capi.raw("llama2_mat_vec", o.ptr, x.ptr, m.ptr, 12, 4) == capi.ERR_INVALID_ARGUMENT
        assert capi.raw("llama2_mat_vec", o.ptr, None, m.ptr, 16, 4) == capi.ERR_INVALID_ARGUMENT
        assert capi.raw("llama2_mat_vec", o.ptr, x.ptr, m.ptr, 16, 4) == capi.OK
        capi.call("llama2_sync")


class TestMatVecStrided:
    def MatVecStrided(self, q, k, dim, n_heads, seq_len):
        head_size = dim // n_heads
        scale = 1.0 / math.sqrt(head_size)
        ip, wt = up(q), up(k)
        att = up(np.zeros(n_heads * seq_len, np.float16))
        capi.call("llama2_mat_vec_strided", att.ptr, ip.ptr, wt.ptr, head_size, seq_len, head_size, head_size, dim,
                  seq_len, scale, n_heads)
        return att.to_host()

    def test_reference_shape(self, oracle):
        # Test_MatVecStrided (test/MatVecStridedTests.cs:74-92): dim 4096, 32 heads, seq 16
        rng = synth.rng_for(211)
        dim, heads, seq = 4096, 32, 16
        q, k = f16(rng.random(dim)), f16(rng.random(dim * heads))
        expected = oracle.ref_matvec_strided(q, k, dim, heads, heads, seq)
        actual = self.MatVecStrided(q, k, dim, heads, seq)
        assert ulp_diff(actual, expected).max() <= 1

    @pytest.mark.parametrize("dim,heads,seq", [(4096, 32, 512), (4096, 32, 2048), (4096, 32, 4096),
                                               (5120, 40, 777), (4096, 32, 1), (512, 2, 33), (4096, 32, 100), (4096, 32, 511),
                                               (4096, 32, 513), (5120, 40, 383)])
    def test_vs_fp64(self, oracle, dim, heads, seq):
        rng = synth.rng_for(212, dim, seq)
        hs = dim // heads
        q, k = synth.normal_f16(rng, dim), synth.normal_f16(rng, seq * dim)
        want = oracle.f64_matvec_strided(q, k, hs, seq, hs, hs, dim, seq, 1 / math.sqrt(hs), heads)
        assert_close(self.MatVecStrided(q, k, dim, heads, seq), want, "scores %d/%d/%d" % (dim, heads, seq))

    def test_generic_strides(self, oracle):
        # head_size 4 (the reference's RoPE test geometry) and odd strides take the generic kernel
        rng = synth.rng_for(213)
        heads, hs, seq, row = 5, 4, 9, 23
        q, k = synth.normal_f16(rng, heads * 6), synth.normal_f16(rng, seq * row)
        att, dq, dk = up(np.zeros(heads * 11, np.float16)), up(q), up(k)
        capi.call("llama2_mat_vec_strided", att.ptr, dq.ptr, dk.ptr, hs, seq, 6, 4, row, 11, 0.5, heads)
        want = oracle.f64_matvec_strided(q, k, hs, seq, 6, 4, row, 11, 0.5, heads)
        got = att.to_host()
        mask = (np.arange(heads * 11) % 11) < seq
        assert_close(got[mask], want[mask], "generic scores")
        assert not got[~mask].any()


class TestVecMat:
    def VecMat(self, att, v, dim, n_heads, seq_len):
        head_size = dim // n_heads
        m, vv = up(att), up(v)
        result = up(np.zeros(dim, np.float16))
        capi.call("llama2_vec_mat", result.ptr, m.ptr, vv.ptr, head_size, seq_len, head_size, head_size, dim, n_heads)
        return result.to_host()

    def test_reference_shape(self, oracle):
        # Test_VecMat (test/VecMatTests.cs:75-93): dim 4096, 32 heads, seq 16
        rng = synth.rng_for(221)
        dim, heads, seq = 4096, 32, 16
        att, v = f16(rng.random(dim)), f16(rng.random(dim * heads))
        expected = oracle.ref_vecmat(att, v, dim, heads, heads, seq)
        actual = self.VecMat(att, v, dim, heads, seq)
        assert ulp_diff(actual, expected).max() <= 1

    @pytest.mark.parametrize("dim,heads,seq", [(4096, 32, 512), (4096, 32, 2048), (4096, 32, 4096),
                                               (5120, 40, 777), (4096, 32, 1), (512, 2, 33), (4096, 32, 100), (4096, 32, 511),
                                               (4096, 32, 513), (5120, 40, 383)])
    def test_vs_fp64(self, oracle, dim, heads, seq):
        rng = synth.rng_for(222, dim, seq)
        hs = dim // heads
        p = rng.random(heads * seq).astype(np.float32).reshape(heads, seq)
        att = f16((p / p.sum(1, keepdims=True)).ravel())
        v = synth.normal_f16(rng, seq * dim)
        want = oracle.f64_vecmat(att, v, hs, seq, hs, hs, dim, heads)
        assert_close(self.VecMat(att, v, dim, heads, seq), want, "vecmat %d/%d/%d" % (dim, heads, seq))

    def test_deterministic(self):
        rng = synth.rng_for(223)
        dim, heads, seq = 4096, 32, 3000
        att, v = f16(rng.random(heads * seq) / seq), synth.normal_f16(rng, seq * dim)
        a = self.VecMat(att, v, dim, heads, seq)
        b = self.VecMat(att, v, dim, heads, seq)
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16))

    def test_generic_strides(self, oracle):
        rng = synth.rng_for(224)
        heads, hs, seq, row = 3, 6, 10, 25
        att, v = f16(rng.random(heads * seq)), synth.normal_f16(rng, seq * row)
        out, datt, dv = up(np.zeros(heads * 7, np.float16)), up(att), up(v)
        capi.call("llama2_vec_mat", out.ptr, datt.ptr, dv.ptr, hs, seq, 6, 7, row, heads)
        want = oracle.f64_vecmat(att, v, hs, seq, 6, 7, row, heads)
        got = out.to_host()
        mask = (np.arange(heads * 7) % 7) < hs
        assert_close(got[mask], want[mask], "generic vecmat")
