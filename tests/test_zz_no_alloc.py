"""GPU check of llama2_vec_mat_static, the VecMat entry point that allocates nothing (the fp32 partial
sums of a sequence split over workgroups live in a file-scope device array of the library), against
llama2_vec_mat: same kernels, so the outputs must agree bit for bit.  Two calls in a row share the
array; the second is smaller and must not be disturbed by what the first left behind."""
import numpy as np
import pytest

from managedllama2_amd import capi, synth
from gpu_util import up

pytestmark = pytest.mark.gpu

HS = 128


def run(name, att, v, dim, heads, seq, expect=capi.OK):
    datt, dv = up(att), up(v)
    out = up(np.zeros(dim, np.float16))
    print("calling %s heads=%d seq=%d dim=%d" % (name, heads, seq, dim), flush=True)
    rc = capi.raw(name, out.ptr, datt.ptr, dv.ptr, HS, seq, HS, HS, dim, heads)
    assert rc == expect, (rc, capi.last_error())
    res = out.to_host()[:heads * HS].view(np.uint16).copy()
    for b in (datt, dv, out):
        b.free()
    return res


def inputs(seed, dim, heads, seq):
    rng = synth.rng_for(seed, dim, seq)
    att = rng.random(heads * seq).astype(np.float32)
    att /= att.reshape(heads, seq).sum(axis=1).repeat(seq)  # rows of softmax-like weights
    return att.astype(np.float16), synth.normal_f16(rng, seq * dim)


def test_static_matches_allocating_entry_point_twice_in_a_row():
    dim, heads = 4096, 32
    a1, v1 = inputs(811, dim, heads, 3000)
    a2, v2 = inputs(812, dim, heads, 700)
    first = run("llama2_vec_mat_static", a1, v1, dim, heads, 3000)   # split over many workgroups: uses the scratch
    second = run("llama2_vec_mat_static", a2, v2, dim, heads, 700)   # fewer, shorter blocks in the same scratch
    assert np.array_equal(first, run("llama2_vec_mat", a1, v1, dim, heads, 3000))
    assert np.array_equal(second, run("llama2_vec_mat", a2, v2, dim, heads, 700))
    assert first.any() and second.any()
    # and again after the allocating entry point ran in between
    assert np.array_equal(first, run("llama2_vec_mat_static", a1, v1, dim, heads, 3000))


def test_static_without_scratch_and_other_head_counts():
    for dim, heads, seq in [(4096, 32, 100), (5120, 40, 777), (512, 3, 1100), (4096, 32, 4096)]:
        a, v = inputs(813, dim, heads, seq)
        assert np.array_equal(run("llama2_vec_mat_static", a, v, dim, heads, seq),
                              run("llama2_vec_mat", a, v, dim, heads, seq)), (dim, heads, seq)


def test_static_rejects_what_does_not_fit():
    # 40 heads x 128 rows x 103 sequence blocks of partial sums = 2.1 MB > LLAMA2_STATIC_VEC_MAT_BYTES;
    # the buffers are real and of full size: whatever the call decides, nothing is read out of bounds
    dim, heads, seq = 5120, 40, 4096
    a, v = inputs(814, dim, heads, seq)
    run("llama2_vec_mat_static", a, v, dim, heads, seq, expect=capi.ERR_UNSUPPORTED)
    assert "static scratch" in capi.last_error()
    run("llama2_vec_mat", a, v, dim, heads, seq)  # the allocating entry point takes it
