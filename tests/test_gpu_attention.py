"""GPU parity of llama2_multi_head_attention -- MultiHeadAttention of the
reference (src/Transformer.cs:150-156: MatVecStrided, Softmax, VecMat) as one
launch -- against the fp64 oracle's composition of the same three steps and
against the three module launches on the GPU.

The reference stores the scaled scores as fp16 before the softmax; the oracle
chain does the same (round_d2h), so both sides exponentiate the same numbers
up to a score whose fp32 and fp64 sums round to different fp16 neighbours.
The softmax weights themselves stay fp32 in the fused kernel (the reference
rounds them to fp16 as well); that difference is below the 2e-3 bound.

Sequence lengths straddle the 512-row block of the kernel: up to 512 rows a
head is one workgroup, beyond that the blocks of a head are merged by the
workgroup that finishes last.
"""
import math

import numpy as np
import pytest

from managedllama2_amd import capi, synth
from gpu_util import assert_close, assert_close_normwise, up

pytestmark = pytest.mark.gpu

HS = 128


def fused(q, k, v, dim, heads, seq):
    dq, dk, dv = up(q), up(k), up(v)
    out = up(np.zeros(dim, np.float16))
    capi.call("llama2_multi_head_attention", out.ptr, dq.ptr, dk.ptr, dv.ptr, HS, dim, seq, 1.0 / math.sqrt(HS), heads)
    return out.to_host()[:heads * HS]


def modules(q, k, v, dim, heads, seq):
    dq, dk, dv = up(q), up(k), up(v)
    att = up(np.zeros(heads * seq, np.float16))
    out = up(np.zeros(dim, np.float16))
    capi.call("llama2_mat_vec_strided", att.ptr, dq.ptr, dk.ptr, HS, seq, HS, HS, dim, seq, 1.0 / math.sqrt(HS), heads)
    capi.call("llama2_softmax", att.ptr, seq, heads)
    capi.call("llama2_vec_mat", out.ptr, att.ptr, dv.ptr, HS, seq, HS, HS, dim, heads)
    return out.to_host()[:heads * HS]


def oracle_chain(oracle, q, k, v, dim, heads, seq):
    scores = oracle.f64_matvec_strided(q, k, HS, seq, HS, HS, dim, seq, 1.0 / math.sqrt(HS), heads)
    p = oracle.f64_softmax(oracle.round_d2h(scores), seq, heads)
    # the fp64 weighted sum, written out here: f64_vecmat takes fp16 weights
    vv = v.astype(np.float64).reshape(seq, dim)[:, :heads * HS].reshape(seq, heads, HS)
    return np.einsum("ht,thj->hj", p.reshape(heads, seq), vv).ravel()


def inputs(seed, dim, seq):
    rng = synth.rng_for(seed, dim, seq)
    return synth.normal_f16(rng, dim), synth.normal_f16(rng, seq * dim), synth.normal_f16(rng, seq * dim)


@pytest.mark.parametrize("dim,heads,seq", [(4096, 32, 1), (4096, 32, 2), (4096, 32, 100), (4096, 32, 511),
                                           (4096, 32, 512), (4096, 32, 513), (4096, 32, 1025), (4096, 32, 3000),
                                           (5120, 40, 777), (512, 3, 1100), (4096, 32, 8192)])
def test_vs_fp64_and_modules(oracle, dim, heads, seq):
    q, k, v = inputs(701, dim, seq)
    got = fused(q, k, v, dim, heads, seq)
    want = oracle_chain(oracle, q, k, v, dim, heads, seq)
    assert_close(got, want, "attention %d/%d/%d" % (dim, heads, seq))
    assert_close_normwise(got, modules(q, k, v, dim, heads, seq), "fused vs modules %d/%d/%d" % (dim, heads, seq))


def test_peaked_scores(oracle):
    """One row dominates the softmax in each block or in a single block: the
    block maxima differ by a lot and the merge must weight them correctly."""
    dim, heads, seq = 512, 4, 1500
    q, k, v = inputs(702, dim, seq)
    k = k.reshape(seq, dim).copy()
    k[3] = (q.astype(np.float32) * 2.0).astype(np.float16)     # large score in block 0
    k[1400] = (q.astype(np.float32) * 1.5).astype(np.float16)  # smaller peak in block 2
    k = k.ravel()
    got = fused(q, k, v, dim, heads, seq)
    want = oracle_chain(oracle, q, k, v, dim, heads, seq)
    assert_close(got, want, "peaked attention")
    # nearly one-hot: the output is close to row 3 of V
    row3 = v.reshape(seq, dim)[3].astype(np.float64)
    assert np.max(np.abs(got.astype(np.float64) - row3)) < 0.05 * np.max(np.abs(row3))


def test_deterministic_and_reusable():
    """The arrival counters return to zero after every launch: repeated calls,
    and calls with a different number of blocks in between, reproduce the bits."""
    dim, heads = 4096, 32
    q, k, v = inputs(703, dim, 3000)
    a = fused(q, k, v, dim, heads, 3000)
    b = fused(q, k, v, dim, heads, 700)
    c = fused(q, k, v, dim, heads, 3000)
    d = fused(q, k, v, dim, heads, 700)
    assert np.array_equal(a.view(np.uint16), c.view(np.uint16))
    assert np.array_equal(b.view(np.uint16), d.view(np.uint16))


def test_rejects_unsupported():
    q, k, v = inputs(704, 512, 4)
    dq, dk, dv, out = up(q), up(k), up(v), up(np.zeros(512, np.float16))
    assert capi.raw("llama2_multi_head_attention", out.ptr, dq.ptr, dk.ptr, dv.ptr, 64, 512, 4, 0.125, 8) == capi.ERR_UNSUPPORTED
    assert capi.raw("llama2_multi_head_attention", out.ptr, dq.ptr, dk.ptr, dv.ptr, HS, 512, 4, 0.1, 5) == capi.ERR_INVALID_ARGUMENT
    assert capi.raw("llama2_multi_head_attention", out.ptr, dq.ptr, dk.ptr, dv.ptr, HS, 512, 0, 0.1, 4) == capi.ERR_INVALID_ARGUMENT
