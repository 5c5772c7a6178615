"""(Kept, skipped and under a name pytest does not collect: see the skip reason below.)

GPU check of llama2_multi_head_attention_static, the attention entry point
that allocates nothing (its partial results and arrival counters live in a
file-scope device array of the library), against llama2_multi_head_attention:
same kernels, so the outputs must agree bit for bit.  Two calls in a row share
the array; the second is smaller and must not see what the first left behind.
Sequence lengths above 128 rows are split into blocks and use the scratch.
"""
import math

import numpy as np
import pytest

pytest.skip("llama2_multi_head_attention_static is not in the library: the one GPU run of an earlier build that "
            "contained it (together with the first version of the persistent decode kernel) ended in a GPU memory "
            "fault, no log of that run came back, and reading the code (every part[] / counters[] index lies inside "
            "the 2 134 016-byte array for every case below) did not show a cause.  The case stays off the GPU; the "
            "entry point that allocates nothing is llama2_vec_mat_static (tests/test_zz_no_alloc.py).",
            allow_module_level=True)

from managedllama2_amd import capi, synth
from gpu_util import up

pytestmark = pytest.mark.gpu

HS = 128


def run(name, q, k, v, dim, heads, seq):
    dq, dk, dv = up(q), up(k), up(v)
    out = up(np.zeros(dim, np.float16))
    capi.call(name, out.ptr, dq.ptr, dk.ptr, dv.ptr, HS, dim, seq, 1.0 / math.sqrt(HS), heads)
    return out.to_host()[:heads * HS].view(np.uint16)


def inputs(seed, dim, seq):
    rng = synth.rng_for(seed, dim, seq)
    return synth.normal_f16(rng, dim), synth.normal_f16(rng, seq * dim), synth.normal_f16(rng, seq * dim)


def test_static_matches_allocating_entry_point_twice_in_a_row():
    dim, heads = 4096, 32
    q, k, v = inputs(811, dim, 3000)
    first = run("llama2_multi_head_attention_static", q, k, v, dim, heads, 3000)   # 24 blocks per head
    second = run("llama2_multi_head_attention_static", q, k, v, dim, heads, 700)   # 6 blocks per head
    third = run("llama2_multi_head_attention_static", q, k, v, dim, heads, 4000)   # 512-row blocks
    assert np.array_equal(first, run("llama2_multi_head_attention", q, k, v, dim, heads, 3000))
    assert np.array_equal(second, run("llama2_multi_head_attention", q, k, v, dim, heads, 700))
    assert np.array_equal(third, run("llama2_multi_head_attention", q, k, v, dim, heads, 4000))
    assert first.any() and second.any() and not np.array_equal(first, second)


def test_static_single_block_and_other_head_counts():
    for dim, heads, seq in [(4096, 32, 100), (5120, 40, 777), (512, 3, 1100)]:
        q, k, v = inputs(812, dim, seq)
        a = run("llama2_multi_head_attention_static", q, k, v, dim, heads, seq)
        b = run("llama2_multi_head_attention", q, k, v, dim, heads, seq)
        assert np.array_equal(a, b), (dim, heads, seq)


def test_static_rejects_what_does_not_fit():
    # 512 heads x 16 blocks of 128 rows = 8192 (head, block) pairs > 4096
    heads, seq = 512, 2048
    dim = heads * HS
    q = up(np.zeros(dim, np.float16))
    kv = up(np.zeros(16, np.float16))  # never read: the call is rejected on the host
    out = up(np.zeros(dim, np.float16))
    rc = capi.raw("llama2_multi_head_attention_static", out.ptr, q.ptr, kv.ptr, kv.ptr, HS, dim, seq, 0.1, heads)
    assert rc == capi.ERR_UNSUPPORTED
    assert "static scratch" in capi.last_error()
    rc = capi.raw("llama2_multi_head_attention_static", out.ptr, q.ptr, kv.ptr, kv.ptr, 64, dim, seq, 0.1, heads)
    assert rc == capi.ERR_UNSUPPORTED
