"""GPU parity of the AWQ int4 mat-vec family through the C ABI, laid out like
the reference's MatVecInt4Tests / QKVMatVecInt4Tests / SwiGLUMatVecInt4Tests
(GPU result vs. CPU `Expected`), plus what those tests leave open: non-zero
zero-points and non-unit scales through the kernels, K = 11008 / 13824
(per-row zero-word padding), full 7B / 13B shapes."""
import numpy as np
import pytest

from managedllama2_amd import capi, synth
from gpu_util import assert_close, sizes, ulp_diff, up, upq, TOL

pytestmark = pytest.mark.gpu


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16)


def reference_regime(rng, K, N, lo=0, hi=15, scale=1.0):
    """test/MatVecInt4Tests.cs:72-80: w in {lo..hi-1}*scale packed with
    HostQWeight.Pack, scales = scale, zeros = 0, x uniform [0,1)."""
    from oracle import oracle
    w = f16(rng.integers(lo, hi, K * N) * scale)
    n_groups = K * N // 128
    W, _, S = oracle.ref_qweight_pack(w, np.full(n_groups, scale, np.float32), np.zeros(n_groups, np.uint32))
    # zeros are 0: the per-row layout wants zeros_size words per row (the flat
    # HostQWeight array the reference test uploads is shorter, see its K=128 case)
    Z = np.zeros(N * synth.qweight_sizes(K)[2], np.uint32)
    x = f16(rng.random(K))
    return (W, Z, S), x


class TestMatVecInt4:
    def MatVecInt4(self, q, x, res, rows, cols):
        zs, ss, ws = sizes(rows)
        dq, dx, dout = upq(q), up(x), up(res)
        capi.call("llama2_mat_vec_residual_int4", dout.ptr, dx.ptr, dq.Weight.ptr, dq.Zeros.ptr, dq.Scales.ptr,
                  rows, cols, zs, ss, ws)
        return dout.to_host()

    def test_reference_regime_exact(self, oracle):
        # Test_MatVecInt4 (test/MatVecInt4Tests.cs:82-93), with the residual in a
        # separate buffer (the reference aliases input and output)
        rng = synth.rng_for(101)
        q, x = reference_regime(rng, 128, 128)
        res = f16(rng.random(128))
        expected = oracle.ref_matvec_residual_int4(res, x, *q, 128, 128)
        actual = self.MatVecInt4(q, x, res, 128, 128)
        assert ulp_diff(actual, expected).max() <= 1
        assert np.mean(actual.view(np.uint16) == expected.view(np.uint16)) >= 0.97

    @pytest.mark.parametrize("K,N", [(4096, 4096), (11008, 4096), (5120, 5120), (13824, 5120), (128, 128),
                                     (256, 7), (4096, 13)])
    def test_random_weights_vs_fp64(self, oracle, K, N):
        rng = synth.rng_for(102, K, N)
        q = synth.random_qweight(rng, K, N)
        x = synth.normal_f16(rng, K)
        res = synth.normal_f16(rng, N)
        want = oracle.f64_matvec_int4(x, *q, K, N) + res.astype(np.float64)
        assert_close(self.MatVecInt4(q, x, res, K, N), want, "residual int4 %dx%d" % (K, N))

    def test_residual_minus_plain(self, oracle):
        rng = synth.rng_for(103)
        K, N = 4096, 512
        q = synth.random_qweight(rng, K, N)
        x = synth.normal_f16(rng, K)
        zs, ss, ws = sizes(K)
        dq, dx = upq(q), up(x)
        plain = up(np.zeros(N, np.float16))
        capi.call("llama2_mat_vec_int4", plain.ptr, dx.ptr, dq.Weight.ptr, dq.Zeros.ptr, dq.Scales.ptr, K, N, zs, ss, ws)
        zero_res = self.MatVecInt4(q, x, np.zeros(N, np.float16), K, N)
        assert np.array_equal(plain.to_host().view(np.uint16), zero_res.view(np.uint16))

    def test_zero_padding_nibbles_are_ignored(self, oracle):
        rng = synth.rng_for(104)
        K, N = 11008, 64
        W, Z, S = synth.random_qweight(rng, K, N)
        x = synth.normal_f16(rng, K)
        res = np.zeros(N, np.float16)
        a = self.MatVecInt4((W, Z, S), x, res, K, N)
        ws, ss, zs = synth.qweight_sizes(K)
        Z2 = Z.reshape(N, zs).copy()
        Z2[:, -1] ^= np.uint32(0xFFFFFFFF) << np.uint32(4 * (ss % 8))
        b = self.MatVecInt4((W, Z2.ravel(), S), x, res, K, N)
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16))

    def test_linearity(self, oracle):
        rng = synth.rng_for(105)
        K, N = 4096, 256
        q = synth.random_qweight(rng, K, N)
        x1 = f16(rng.integers(-3, 4, K))
        x2 = f16(rng.integers(-3, 4, K))
        z = np.zeros(N, np.float16)
        y1 = self.MatVecInt4(q, x1, z, K, N).astype(np.float64)
        y2 = self.MatVecInt4(q, x2, z, K, N).astype(np.float64)
        y12 = self.MatVecInt4(q, f16(x1.astype(np.float32) + x2.astype(np.float32)), z, K, N).astype(np.float64)
        # each of the three results carries its own fp16 rounding (2^-11 relative)
        bound = 2.0 ** -10 * (np.abs(y1) + np.abs(y2) + np.abs(y12)) + 1e-6
        assert np.all(np.abs(y12 - (y1 + y2)) <= bound)

    def test_argument_errors(self):
        rng = synth.rng_for(106)
        K, N = 128, 8
        q = upq(synth.random_qweight(rng, K, N))
        x, out = up(synth.normal_f16(rng, K)), up(np.zeros(N, np.float16))
        zs, ss, ws = sizes(K)
        args = [out.ptr, x.ptr, q.Weight.ptr, q.Zeros.ptr, q.Scales.ptr, K, N, zs, ss, ws]
        assert capi.raw("llama2_mat_vec_residual_int4", *args) == capi.OK
        bad = list(args); bad[9] = ws + 4
        assert capi.raw("llama2_mat_vec_residual_int4", *bad) == capi.ERR_INVALID_ARGUMENT
        assert "sizes" in capi.last_error()
        bad = list(args); bad[2] = None
        assert capi.raw("llama2_mat_vec_residual_int4", *bad) == capi.ERR_INVALID_ARGUMENT
        bad = list(args); bad[2] = q.Weight.ptr + 4
        assert capi.raw("llama2_mat_vec_residual_int4", *bad) == capi.ERR_INVALID_ARGUMENT
        bad = list(args); bad[0] = x.ptr  # in place: rejected (races in the reference's own test)
        assert capi.raw("llama2_mat_vec_residual_int4", *bad) == capi.ERR_INVALID_ARGUMENT
        bad = list(args); bad[5] = 0
        assert capi.raw("llama2_mat_vec_residual_int4", *bad) == capi.ERR_INVALID_ARGUMENT
        capi.call("llama2_sync")


class TestQKVMatVecInt4:
    def QKVMatVecInt4(self, xb, qw, kw, vw, rows, cols):
        zs, ss, ws = sizes(rows)
        dx = up(xb)
        dq, dk, dv = upq(qw), upq(kw), upq(vw)
        outs = [up(np.zeros(cols, np.float16)) for _ in range(3)]
        capi.call("llama2_qkv_mat_vec", outs[0].ptr, outs[1].ptr, outs[2].ptr, dx.ptr,
                  dq.Weight.ptr, dq.Zeros.ptr, dq.Scales.ptr, dk.Weight.ptr, dk.Zeros.ptr, dk.Scales.ptr,
                  dv.Weight.ptr, dv.Zeros.ptr, dv.Scales.ptr, rows, cols, zs, ss, ws)
        return [o.to_host() for o in outs]

    def test_reference_regime_exact(self, oracle):
        # Test_QKVMatVecInt4 (test/QKVMatVecInt4Tests.cs:103-119)
        rng = synth.rng_for(111)
        x = f16(rng.random(128))
        qs = [reference_regime(rng, 128, 128)[0] for _ in range(3)]
        actual = self.QKVMatVecInt4(x, *qs, 128, 128)
        for a, q in zip(actual, qs):
            expected = oracle.ref_matvec_int4(x, *q, 128, 128)
            assert ulp_diff(a, expected).max() <= 1
            assert np.mean(a.view(np.uint16) == expected.view(np.uint16)) >= 0.97

    @pytest.mark.parametrize("dim", [4096, 5120])
    def test_fused_equals_three_plain_and_fp64(self, oracle, dim):
        rng = synth.rng_for(112, dim)
        qs = [synth.random_qweight(rng, dim, dim) for _ in range(3)]
        x = synth.normal_f16(rng, dim)
        actual = self.QKVMatVecInt4(x, *qs, dim, dim)
        zs, ss, ws = sizes(dim)
        dx = up(x)
        for a, q in zip(actual, qs):
            assert_close(a, oracle.f64_matvec_int4(x, *q, dim, dim), "qkv %d" % dim)
            dq, o = upq(q), up(np.zeros(dim, np.float16))
            capi.call("llama2_mat_vec_int4", o.ptr, dx.ptr, dq.Weight.ptr, dq.Zeros.ptr, dq.Scales.ptr, dim, dim, zs, ss, ws)
            assert np.array_equal(o.to_host().view(np.uint16), a.view(np.uint16))


class TestSwiGLUMatVecInt4:
    def SwiGLUMatVecInt4(self, g, u, x, rows, cols):
        zs, ss, ws = sizes(rows)
        dg, du, dx = upq(g), upq(u), up(x)
        out = up(np.zeros(cols, np.float16))
        capi.call("llama2_mat_vec_swiglu", out.ptr, dx.ptr, dg.Weight.ptr, dg.Zeros.ptr, dg.Scales.ptr,
                  du.Weight.ptr, du.Zeros.ptr, du.Scales.ptr, rows, cols, zs, ss, ws)
        return out.to_host()

    def test_reference_regime(self, oracle):
        # Test_SwiGLUMatVecInt4 (test/SwiGLUMatVecInt4Tests.cs:94-122): the reference
        # compares Half.Truncate of both sides; here additionally 2e-3
        rng = synth.rng_for(121)
        g, x = reference_regime(rng, 128, 128, 0, 15, 0.01)
        u, _ = reference_regime(rng, 128, 128, 0, 15, 0.01)
        expected = oracle.ref_matvec_swiglu(x, g, u, 128, 128)
        actual = self.SwiGLUMatVecInt4(g, u, x, 128, 128)
        assert np.array_equal(np.trunc(actual.astype(np.float32)), np.trunc(expected.astype(np.float32)))
        assert_close(actual, expected.astype(np.float64), "swiglu reference regime")

    @pytest.mark.parametrize("K,N", [(4096, 11008), (5120, 13824), (256, 10)])
    def test_random_weights_vs_fp64(self, oracle, K, N):
        rng = synth.rng_for(122, K, N)
        g = synth.random_qweight(rng, K, N)
        u = synth.random_qweight(rng, K, N)
        # x ~ N(0, 1) like every other mat-vec test: |gate| and |up| reach about 20, silu(g) * u a few
        # hundred, far inside the fp16 range
        x = synth.normal_f16(rng, K)
        gv = oracle.f64_matvec_int4(x, *g, K, N)
        uv = oracle.f64_matvec_int4(x, *u, K, N)
        want = gv / (1 + np.exp(-gv)) * uv
        assert_close(self.SwiGLUMatVecInt4(g, u, x, K, N), want, "swiglu %dx%d" % (K, N))
