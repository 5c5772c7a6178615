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


MAX_TIE_FRACTION = 0.025  # of all scores may take the tie slack (measured: 1.6 .. 1.8 % at 100 .. 8192 rows)
TIES = []   # (scores that took the tie slack, scores) of every oracle_chain(..., with_slack=True) call
TIE = 1e-6  # a score this close to the midpoint of two fp16 values may round either way (fp32 sum of 128 products)


def oracle_chain(oracle, q, k, v, dim, heads, seq, with_slack=False):
    """fp64 scores, rounded to fp16 as the reference stores them, fp64 softmax and weighted sum.
    with_slack: also returns, per output, how far it moves if every score within TIE of a rounding
    midpoint had rounded the other way (the weight of that row changes by one fp16 step of its
    score): the fp32 sum on the GPU and the fp64 sum here cannot agree on those."""
    scores = oracle.f64_matvec_strided(q, k, HS, seq, HS, HS, dim, seq, 1.0 / math.sqrt(HS), heads)
    rounded = oracle.round_d2h(scores)
    p = oracle.f64_softmax(rounded, seq, heads).reshape(heads, seq)
    # the fp64 weighted sum, written out here: f64_vecmat takes fp16 weights
    vv = v.astype(np.float64).reshape(seq, dim)[:, :heads * HS].reshape(seq, heads, HS)
    out = np.einsum("ht,thj->hj", p, vv)
    if not with_slack:
        return out.ravel()
    r = rounded.astype(np.float64).reshape(heads, seq)
    step = np.abs(np.nextafter(rounded, np.float16(np.inf)).astype(np.float64).reshape(heads, seq) - r)
    step = np.maximum(step, np.abs(r - np.nextafter(rounded, np.float16(-np.inf)).astype(np.float64).reshape(heads, seq)))
    near = (step / 2 - np.abs(scores.reshape(heads, seq) - r)) < TIE
    w = np.where(near, p * step, 0.0)  # d p_t = p_t * d s_t
    slack = np.einsum("ht,thj->hj", w, np.abs(vv)) + w.sum(axis=1)[:, None] * np.abs(out)
    TIES.append((int(near.sum()), near.size))
    return out.ravel(), slack.ravel()


def assert_close_up_to_ties(got, want_slack, what):
    """gpu_util.assert_close (2e-3 with the 2^-8 floor, 4e-3 with the 2^-10 floor) after taking
    the tie slack off the difference."""
    want, slack = want_slack
    n_tie, n_scores = TIES[-1]
    print("%s: %d of %d scores within %g of an fp16 rounding midpoint took the tie slack" % (what, n_tie, n_scores, TIE))
    assert n_tie <= MAX_TIE_FRACTION * n_scores + 2, (what, n_tie, n_scores)
    diff = got.astype(np.float64) - want
    diff = np.sign(diff) * np.maximum(np.abs(diff) - slack, 0.0)
    assert_close(want + diff, want, what)


def inputs(seed, dim, seq):
    rng = synth.rng_for(seed, dim, seq)
    return synth.normal_f16(rng, dim), synth.normal_f16(rng, seq * dim), synth.normal_f16(rng, seq * dim)


@pytest.mark.parametrize("dim,heads,seq", [(4096, 32, 1), (4096, 32, 2), (4096, 32, 100), (4096, 32, 511),
                                           (4096, 32, 512), (4096, 32, 513), (4096, 32, 1025), (4096, 32, 2048),
                                           (4096, 32, 3000), (4096, 32, 3072), (4096, 32, 3073), (4096, 32, 4096),
                                           (5120, 40, 777), (512, 3, 1100), (4096, 32, 8192)])
def test_vs_fp64_and_modules(oracle, dim, heads, seq):
    q, k, v = inputs(701, dim, seq)
    got = fused(q, k, v, dim, heads, seq)
    assert_close_up_to_ties(got, oracle_chain(oracle, q, k, v, dim, heads, seq, True), "attention %d/%d/%d" % (dim, heads, seq))
    assert_close_normwise(got, modules(q, k, v, dim, heads, seq), "fused vs modules %d/%d/%d" % (dim, heads, seq))


def rope_then_attention(q, k, v, dim, heads, seq, pos, one_launch):
    """RoPE at `pos` on the query and on row seq - 1 of K, then attention over seq rows:
    two launches (llama2_rope, llama2_multi_head_attention) or the one-launch entry point.
    Returns (output, rotated query, rotated K row)."""
    dq, dk, dv = up(q), up(k), up(v)
    out = up(np.zeros(dim, np.float16))
    scale = 1.0 / math.sqrt(HS)
    if one_launch:
        capi.call("llama2_rope_multi_head_attention", out.ptr, dq.ptr, dk.ptr, dv.ptr, HS, dim, seq, scale, heads, pos,
                  10000.0)
    else:
        capi.call("llama2_rope", dq.ptr, dk.offset_pointer((seq - 1) * dim), heads, HS, pos, 10000.0, heads)
        capi.call("llama2_multi_head_attention", out.ptr, dq.ptr, dk.ptr, dv.ptr, HS, dim, seq, scale, heads)
    return out.to_host()[:heads * HS], dq.to_host(), dk.to_host(dim, (seq - 1) * dim), dk.to_host(dim, 0)


@pytest.mark.parametrize("seq", [512, 2048, 4096])
def test_rope_then_attention_as_the_decode_step_runs_it(oracle, seq):
    """The attention workload as the reference's step runs it (src/Transformer.cs:172-175): RoPERotation
    at pos = seq on the query and on the newest K row, then MultiHeadAttention over seq rows of a
    32-head, 128-wide fp16 cache.  Three checks:
    (1) the rotated query and K row against the fp64 rotation, within the angle error of the
        reference's fp32 angle (native/rope_kernel.cu:8-12: up to pos * 2^-22 rad) times the
        pair's norm, plus the fp16 rounding;
    (2) the output against the fp64 attention chain fed with the rotated fp16 values the GPU
        stored (the reference stores fp16 there too), element-wise at 2e-3: both sides then
        exponentiate the same fp16 scores, up to scores that sit on a rounding midpoint;
    (3) the output against an fp64 chain that starts from the UNROTATED inputs (fp64 rotation,
        rounded to fp16).  The one-step differences of (1) move the scores before they are
        rounded to fp16, so single scores round the other way and an output near a zero
        crossing moves by more than 2e-3 of ITSELF: this check is norm-wise, 2e-3 of the
        largest output."""
    dim, heads = 4096, 32
    q, k, v = inputs(705, dim, seq)
    got, gq, gk, _ = rope_then_attention(q, k, v, dim, heads, seq, seq, one_launch=False)
    krow = k[(seq - 1) * dim:]
    wq, wk = oracle.f64_rope(q, krow, heads, heads, HS, seq)
    for g, w, src in ((gq, wq, q), (gk, wk, krow)):
        pair = src.astype(np.float64).reshape(heads, 2, HS // 2)
        norm = np.repeat(np.sqrt(pair[:, 0] ** 2 + pair[:, 1] ** 2)[:, None, :], 2, axis=1).reshape(-1)
        assert np.all(np.abs(g.astype(np.float64) - w) <= norm * (seq * 2.0 ** -21 + 2.0 ** -10) + 1e-7)
    kg = k.copy()
    kg[(seq - 1) * dim:] = gk
    assert_close_up_to_ties(got, oracle_chain(oracle, gq, kg, v, dim, heads, seq, True), "rope+attention %d" % seq)
    k64 = k.copy()
    k64[(seq - 1) * dim:] = oracle.round_d2h(wk)
    want = oracle_chain(oracle, oracle.round_d2h(wq), k64, v, dim, heads, seq)
    assert_close_normwise(got, want, "rope + attention from unrotated inputs %d" % seq, 2e-3)


@pytest.mark.parametrize("dim,heads,seq,pos", [(4096, 32, 1, 0), (4096, 32, 100, 99), (4096, 32, 512, 512),
                                               (4096, 32, 513, 512), (4096, 32, 2048, 2048), (4096, 32, 3072, 3071),
                                               (4096, 32, 3073, 3072), (4096, 32, 4096, 4096), (5120, 40, 777, 776),
                                               (512, 3, 1100, 7)])
def test_one_launch_rope_attention_equals_two_launches(dim, heads, seq, pos):
    """llama2_rope_multi_head_attention against llama2_rope + llama2_multi_head_attention: output,
    rotated query and rotated K row bit for bit; no other K row is touched; heads beyond n_heads
    (dim 512 holds 4, 3 are used) keep their query and K columns."""
    q, k, v = inputs(706, dim, seq)
    two = rope_then_attention(q, k, v, dim, heads, seq, pos, one_launch=False)
    one = rope_then_attention(q, k, v, dim, heads, seq, pos, one_launch=True)
    for a, b, what in zip(two, one, ("output", "query", "newest K row", "K row 0")):
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), "%s differs (%d/%d/%d)" % (what, dim, heads, seq)
    if seq > 1:
        assert np.array_equal(one[3].view(np.uint16), k[:dim].view(np.uint16))
    assert not np.array_equal(one[1][:heads * HS].view(np.uint16), q[:heads * HS].view(np.uint16)) or pos == 0
    assert np.array_equal(one[1][heads * HS:].view(np.uint16), q[heads * HS:].view(np.uint16))


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
