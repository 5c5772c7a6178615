"""Pins every operator of the CPU oracle against something that is not the
oracle's own formula: exact integer arithmetic, numpy fp64 matmul on strided
views, brute force in pure Python on small inputs, textbook closed forms and
invariants.  A dropped term, a wrong sign/index or a transposed operand fails
at least one of these."""
import math

import numpy as np
import pytest

from managedllama2_amd import synth


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16)


# ----------------------------------------------------------------- int4 GEMV family
def pack_rows(wint, zint, K, N):
    """Pack integer nibbles [N][K] and per-group zeros [N][K/128] into the
    per-row layout, with garbage in the unused zero nibbles."""
    ws, ss, zs = synth.qweight_sizes(K)
    W = np.zeros((N, ws), np.uint32)
    for i in range(8):
        W[:, : K // 8] |= (wint[:, i::8].astype(np.uint32) & 0xF) << np.uint32(4 * i)
    Z = np.full((N, zs), 0xFFFFFFFF, np.uint32)  # padding nibbles = 0xF: must be ignored
    for g in range(ss):
        Z[:, g // 8] &= ~(np.uint32(0xF) << np.uint32(4 * (g % 8)))
        Z[:, g // 8] |= (zint[:, g].astype(np.uint32) & 0xF) << np.uint32(4 * (g % 8))
    return W.ravel(), Z.ravel()


def test_int4_integer_regime_is_exact(oracle):
    # the reference tests' regime (scale 1, zero 0, test/MatVecInt4Tests.cs:72-80)
    # with small-integer x: every quantity is an exact integer
    rng = np.random.default_rng(7)
    K = N = 128
    w = rng.integers(0, 15, (N, K))
    x = rng.integers(-4, 5, K)
    W, Z = pack_rows(w, np.zeros((N, 1), np.int64), K, N)
    S = np.ones(N, np.float16)
    want = w @ x
    assert np.array_equal(oracle.f64_matvec_int4(f16(x), W, Z, S, K, N), want.astype(np.float64))
    assert np.array_equal(oracle.ref_matvec_int4(f16(x), W, Z, S, K, N), f16(want))
    res = f16(rng.integers(-8, 9, N))
    got = oracle.ref_matvec_residual_int4(res, f16(x), W, Z, S, K, N)
    assert np.array_equal(got, f16(want + res.astype(np.int64)))


def test_int4_brute_force_small(oracle):
    # pure-Python nibble extraction on a 128x256 matrix with non-trivial zeros/scales
    rng = synth.rng_for(11)
    K, N = 256, 128
    W, Z, S = synth.random_qweight(rng, K, N)
    x = synth.normal_f16(rng, K)
    ws, ss, zs = synth.qweight_sizes(K)
    want = []
    for n in range(N):
        acc = 0.0
        for k in range(K):
            wv = (int(W[n * ws + k // 8]) >> (4 * (k % 8))) & 15
            g = k // 128
            zv = (int(Z[n * zs + g // 8]) >> (4 * (g % 8))) & 15
            acc += float(x[k]) * (wv - zv) * float(S[n * ss + g])
        want.append(acc)
    got = oracle.f64_matvec_int4(x, W, Z, S, K, N)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    # C#-style path: within fp16 rounding of weights (2^-11) and of the result
    ref = oracle.ref_matvec_int4(x, W, Z, S, K, N).astype(np.float64)
    assert np.max(np.abs(ref - got)) <= 2e-3 * np.max(np.abs(got))


@pytest.mark.parametrize("K", [11008, 13824])
def test_row_padded_zeros_match_per_row_flat_unpack(oracle, K):
    # K/128 is not a multiple of 8: each row owns ceil(groups/8) zero words.
    # Unpacking every row as its own flat HostQWeight (pinned by the golden
    # vector) must equal the row-layout unpack of the whole tensor.
    rng = synth.rng_for(12, K)
    N = 5
    W, Z, S = synth.random_qweight(rng, K, N)
    ws, ss, zs = synth.qweight_sizes(K)
    assert zs * 8 > ss  # padded
    rows = oracle.ref_qweight_unpack_rows(W, Z, S, K, N)
    for n in range(N):
        flat = oracle.ref_qweight_unpack(W[n * ws:(n + 1) * ws].copy(), Z[n * zs:(n + 1) * zs].copy(),
                                         S[n * ss:(n + 1) * ss].copy())
        assert np.array_equal(rows[n], flat[:K])
    # padding nibbles are don't-care
    Z2 = Z.copy().reshape(N, zs)
    Z2[:, -1] ^= np.uint32(0xFFFFFFFF) << np.uint32(4 * (ss % 8))
    assert np.array_equal(oracle.ref_qweight_unpack_rows(W, Z2.ravel(), S, K, N), rows)
    x = synth.normal_f16(rng, K)
    assert np.array_equal(oracle.f64_matvec_int4(x, W, Z2.ravel(), S, K, N),
                          oracle.f64_matvec_int4(x, W, Z, S, K, N))
    d = oracle.f64_dequant_rows(W, Z, S, K, N)
    assert np.allclose(oracle.f64_matvec_int4(x, W, Z, S, K, N), d @ x.astype(np.float64), rtol=1e-12)
    assert np.array_equal(d.astype(np.float16), rows)


def test_int4_linearity_and_family_identities(oracle):
    rng = synth.rng_for(13)
    K, N = 512, 64
    W, Z, S = synth.random_qweight(rng, K, N)
    x1 = f16(rng.integers(-3, 4, K))
    x2 = f16(rng.integers(-3, 4, K))
    y1 = oracle.f64_matvec_int4(x1, W, Z, S, K, N)
    y2 = oracle.f64_matvec_int4(x2, W, Z, S, K, N)
    y12 = oracle.f64_matvec_int4(f16(x1.astype(np.float32) + x2.astype(np.float32)), W, Z, S, K, N)
    assert np.allclose(y12, y1 + y2, rtol=1e-12, atol=1e-12)
    # SwiGLU == silu(plain gate) * plain up (test/SwiGLUMatVecInt4Tests.cs:75-92)
    g = synth.random_qweight(rng, K, N)
    u = synth.random_qweight(rng, K, N)
    x = synth.normal_f16(rng, K)
    gv = oracle.f64_matvec_int4(x, *g, K, N)
    uv = oracle.f64_matvec_int4(x, *u, K, N)
    want = gv / (1 + np.exp(-gv)) * uv
    got = oracle.ref_matvec_swiglu(x, g, u, K, N).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2e-3 * np.max(np.abs(want))


# ----------------------------------------------------------------- fp16 GEMVs
def test_matvec_f16_vs_numpy(oracle):
    rng = synth.rng_for(14)
    K, N = 4096, 64  # test/MatVecTests.cs:60-62
    M = f16(rng.random(N * K))
    x = f16(rng.random(K))
    want = M.reshape(N, K).astype(np.float64) @ x.astype(np.float64)
    assert np.allclose(oracle.f64_matvec_f16(x, M, K, N), want, rtol=1e-13)
    ref = oracle.ref_matvec(M, x, K, N)
    assert np.max(np.abs(ref.astype(np.float64) - want) / want) < 1e-3


def test_strided_scores_and_vecmat_vs_numpy(oracle):
    rng = synth.rng_for(15)
    dim, heads, S = 512, 8, 16
    hs = dim // heads
    q = synth.normal_f16(rng, dim)
    Kc = synth.normal_f16(rng, 32 * dim)
    alpha = 1 / math.sqrt(hs)
    want = np.einsum("hr,thr->ht", q.reshape(heads, hs).astype(np.float64),
                     Kc.reshape(32, heads, hs)[:S].astype(np.float64)) * alpha
    got = oracle.f64_matvec_strided(q, Kc, hs, S, hs, hs, dim, S, alpha, heads).reshape(heads, S)
    assert np.allclose(got, want, rtol=1e-13, atol=1e-13)
    ref = oracle.ref_matvec_strided(q, Kc, dim, heads, heads, S).reshape(heads, S)
    assert np.max(np.abs(ref.astype(np.float64) - want)) < 2e-3 * np.max(np.abs(want))
    att = f16(rng.random(heads * S))
    wantv = np.einsum("ht,thr->hr", att.reshape(heads, S).astype(np.float64),
                      Kc.reshape(32, heads, hs)[:S].astype(np.float64)).ravel()
    gotv = oracle.f64_vecmat(att, Kc, hs, S, hs, hs, dim, heads)
    assert np.allclose(gotv, wantv, rtol=1e-13, atol=1e-13)
    refv = oracle.ref_vecmat(att, Kc, dim, heads, heads, S)
    assert np.max(np.abs(refv.astype(np.float64) - wantv)) < 2e-3 * np.max(np.abs(wantv))


# ----------------------------------------------------------------- softmax
def test_softmax_closed_forms(oracle):
    two = f16([0.25, 1.5])
    p = oracle.f64_softmax(two, 2, 1)
    assert p[0] == pytest.approx(1 / (1 + math.exp(1.25)), rel=1e-14)
    assert p[1] == pytest.approx(1 / (1 + math.exp(-1.25)), rel=1e-14)
    rng = synth.rng_for(16)
    x = synth.normal_f16(rng, 3 * 50)
    p = oracle.f64_softmax(x, 50, 3).reshape(3, 50)
    assert np.allclose(p.sum(1), 1, rtol=1e-13)
    shifted = f16(x.astype(np.float32) + 2)  # exact for |x| < 6: spacing allows it? use integers
    xi = f16(rng.integers(-6, 7, 40))
    assert np.allclose(oracle.f64_softmax(f16(xi.astype(np.float32) + 3), 40, 1), oracle.f64_softmax(xi, 40, 1),
                       rtol=1e-13)
    assert np.array_equal(np.argsort(p[0], kind="stable"), np.argsort(x[:50].astype(np.float64), kind="stable"))
    r = oracle.ref_softmax(x[:50]).astype(np.float64)
    assert np.max(np.abs(r - p[0])) < 1e-3 * p[0].max()
    del shifted


# ----------------------------------------------------------------- rmsnorm
@pytest.mark.parametrize("v,g", [([1, 2, 3], [4, 5, 6]), ([6, 2, 6], [1, 9, 7])])  # test/RMSNormTests.cs:64-65
def test_rmsnorm_inline_vectors(oracle, v, g):
    r = 1 / math.sqrt(sum(a * a for a in v) / 3 + 1e-5)
    want = f16([gi * vi * r for vi, gi in zip(v, g)])
    assert np.array_equal(oracle.ref_rmsnorm(f16(v), f16(g)), want)
    assert np.array_equal(oracle.ref_rmsnorm(f16(v), f16(g), square_in_half=False), want)
    assert np.allclose(oracle.f64_rmsnorm(f16(v), f16(g)), [gi * vi * r for vi, gi in zip(v, g)], rtol=1e-14)


def test_rmsnorm_unit_rms(oracle):
    rng = synth.rng_for(17)
    x = synth.normal_f16(rng, 4096)
    y = oracle.f64_rmsnorm(x, np.ones(4096, np.float16))
    assert math.sqrt(np.mean(y * y)) == pytest.approx(1.0, abs=1e-4)


# ----------------------------------------------------------------- rope
def test_rope_closed_forms(oracle):
    heads, hs, theta = 4, 128, 10000.0
    dim = heads * hs
    rng = synth.rng_for(18)
    q = synth.normal_f16(rng, dim)
    k = synth.normal_f16(rng, dim)
    q0, k0 = oracle.f64_rope(q, k, heads, heads, hs, 0, theta)
    assert np.array_equal(q0, q.astype(np.float64)) and np.array_equal(k0, k.astype(np.float64))
    rq, rk = oracle.ref_rope(q, k, dim, heads, heads, 0, theta)
    assert np.array_equal(rq, q) and np.array_equal(rk, k)
    pos = 37
    qr, kr = oracle.f64_rope(q, k, heads, heads, hs, pos, theta)
    a = qr.reshape(heads, 2, hs // 2)
    b = q.astype(np.float64).reshape(heads, 2, hs // 2)
    assert np.allclose(a[:, 0] ** 2 + a[:, 1] ** 2, b[:, 0] ** 2 + b[:, 1] ** 2, rtol=1e-12)
    # unit vector in slot t of every head rotates to (cos, sin)(pos * theta^(-2t/hs)) in (t, t+hs/2)
    for t in (0, 1, 17, 63):
        e = np.zeros(dim, np.float16)
        e[np.arange(heads) * hs + t] = 1
        qe, ke = oracle.f64_rope(e, e, heads, heads, hs, pos, theta)
        ang = pos * theta ** (-2 * t / hs)
        for h in range(heads):
            assert qe[h * hs + t] == pytest.approx(math.cos(ang), abs=1e-12)
            assert qe[h * hs + t + hs // 2] == pytest.approx(math.sin(ang), abs=1e-12)
            assert ke[h * hs + t] == pytest.approx(math.cos(ang), abs=1e-12)
        assert np.count_nonzero(qe) == 2 * heads
    # fewer kv heads: only the first n_kv_heads heads of k rotate (native/rope_kernel.cu:19)
    qr2, kr2 = oracle.f64_rope(q, k, heads, 2, hs, pos, theta)
    assert np.array_equal(kr2[: 2 * hs], kr[: 2 * hs]) and not kr2[2 * hs:].any()
    # fp32 restatement agrees with fp64 to fp16 rounding
    rq, rk = oracle.ref_rope(q, k, dim, heads, heads, pos, theta)
    assert np.max(np.abs(rq.astype(np.float64) - qr)) < 4e-3
    assert np.max(np.abs(rk.astype(np.float64) - kr)) < 4e-3


# ----------------------------------------------------------------- argmax / embedding
def test_argmax_first_maximum(oracle):
    rng = synth.rng_for(19)
    x = f16(rng.random(32000))
    assert oracle.ref_argmax(x) == int(np.argmax(x))
    x[[5, 100, 31999]] = 2.0  # ties: lowest index wins (strict '>')
    assert oracle.ref_argmax(x) == 5
    assert oracle.ref_argmax(f16([-3, -1, -1, -2])) == 1


def test_embedding_row_copy(oracle):
    rng = synth.rng_for(20)
    table = f16(rng.random(7 * 256))
    tokens = np.array([3, 0, 6], np.int32)
    assert np.array_equal(oracle.ref_embedding(table, 256, tokens, 2), table[6 * 256:7 * 256])
    assert np.array_equal(oracle.ref_embedding(table, 256, tokens, 1), table[:256])


# ----------------------------------------------------------------- one decode step
def test_forward_composition(oracle):
    """f64_forward equals the modules applied in the order of
    src/Transformer.cs:158-190, including the KV-cache row written at
    layerOffset + pos*kvDim and attention over pos+1 rows."""
    cfg = dict(dim=256, hidden_dim=384, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=320,
               seq_len=8, rope_theta=10000.0)
    model = synth.random_model(cfg, seed=3, rms_random=True)
    hm = oracle.HostModel(cfg, model)
    hm.tokens[:3] = [5, 17, 300]
    dim, hd, H, S = cfg["dim"], cfg["hidden_dim"], cfg["n_heads"], cfg["seq_len"]
    hs = dim // H
    kc = np.zeros((cfg["n_layers"], S, dim), np.float16)
    vc = np.zeros((cfg["n_layers"], S, dim), np.float16)
    r = oracle.round_d2h
    for pos in range(3):
        logits = hm.forward(pos, pos + 1).copy()
        x = model["embedding"][hm.tokens[pos] * dim:(hm.tokens[pos] + 1) * dim].copy()
        for l, L in enumerate(model["layers"]):
            xb = r(oracle.f64_rmsnorm(x, L["rms_att"]))
            q = r(oracle.f64_matvec_int4(xb, *L["q"], dim, dim))
            k = r(oracle.f64_matvec_int4(xb, *L["k"], dim, dim))
            v = r(oracle.f64_matvec_int4(xb, *L["v"], dim, dim))
            qd, kd = oracle.f64_rope(q, k, H, H, hs, pos, 10000.0)
            q, kc[l, pos], vc[l, pos] = r(qd), r(kd), v
            n = pos + 1
            att = r(oracle.f64_matvec_strided(q, kc[l].ravel(), hs, n, hs, hs, dim, n, 1 / math.sqrt(hs), H))
            att = r(oracle.f64_softmax(att, n, H))
            xb = r(oracle.f64_vecmat(att, vc[l].ravel(), hs, n, hs, hs, dim, H))
            x = r(oracle.f64_matvec_int4(xb, *L["o"], dim, dim) + x.astype(np.float64))
            xb = r(oracle.f64_rmsnorm(x, L["rms_ffn"]))
            g = oracle.f64_matvec_int4(xb, *L["gate"], dim, hd)
            u = oracle.f64_matvec_int4(xb, *L["up"], dim, hd)
            h = r(g / (1 + np.exp(-g)) * u)
            x = r(oracle.f64_matvec_int4(h, *L["down"], hd, dim) + x.astype(np.float64))
        x = r(oracle.f64_rmsnorm(x, model["rms_final"]))
        want = r(oracle.f64_matvec_f16(x, model["classifier"], dim, cfg["vocab_size"]))
        assert np.array_equal(logits, want), pos
        assert np.array_equal(hm.key_cache.reshape(kc.shape), kc)
        assert np.array_equal(hm.value_cache.reshape(vc.shape), vc)
    assert np.isfinite(logits.astype(np.float32)).all() and logits.astype(np.float32).std() > 0
