"""Seeded int4 mat-vec results through the C ABI, as a dictionary of fp16 arrays: the same call in two
processes (one with an environment switch that changes which kernel the launcher picks) must give
the same bits.  Not a test module by itself (pytest does not collect it)."""
import numpy as np

from managedllama2_amd import capi, synth
from gpu_util import sizes, up, upq

SHAPES = [(4096, 4096), (4096, 1000), (4096, 11008), (11008, 4096), (5120, 5120), (13824, 5120), (256, 7),
          (4096, 13), (2048, 333)]


def run_all():
    out = {}
    for K, N in SHAPES:
        rng = synth.rng_for(991, K, N)
        zs, ss, ws = sizes(K)
        x = up(synth.normal_f16(rng, K))
        qs = [upq(synth.random_qweight(rng, K, N)) for _ in range(3)]
        res = synth.normal_f16(rng, N)
        o = [up(res.copy()) for _ in range(3)]
        capi.call("llama2_mat_vec_int4", o[0].ptr, x.ptr, qs[0].Weight.ptr, qs[0].Zeros.ptr, qs[0].Scales.ptr, K, N, zs, ss, ws)
        out["plain_%dx%d" % (K, N)] = o[0].to_host()
        capi.call("llama2_mat_vec_residual_int4", o[1].ptr, x.ptr, qs[1].Weight.ptr, qs[1].Zeros.ptr, qs[1].Scales.ptr,
                  K, N, zs, ss, ws)
        out["residual_%dx%d" % (K, N)] = o[1].to_host()
        capi.call("llama2_mat_vec_swiglu", o[2].ptr, x.ptr, qs[0].Weight.ptr, qs[0].Zeros.ptr, qs[0].Scales.ptr,
                  qs[1].Weight.ptr, qs[1].Zeros.ptr, qs[1].Scales.ptr, K, N, zs, ss, ws)
        out["swiglu_%dx%d" % (K, N)] = o[2].to_host()
        if K == N:
            capi.call("llama2_qkv_mat_vec", o[0].ptr, o[1].ptr, o[2].ptr, x.ptr,
                      *[p for q in qs for p in (q.Weight.ptr, q.Zeros.ptr, q.Scales.ptr)], K, N, zs, ss, ws)
            for name, buf in zip("qkv", o):
                out["qkv_%s_%d" % (name, K)] = buf.to_host()
        for b in o + [x]:
            b.free()
        for q in qs:
            for b in (q.Weight, q.Zeros, q.Scales):
                b.free()
    return out
