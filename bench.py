#!/usr/bin/env python3
"""Benchmark of the quantized batch-1 decode hot path on one MI355X.

A "step" is one Llama-2-7B decoder layer's int4 mat-vec set at batch 1 (fused
QKV 3x4096x4096, o-proj 4096x4096 + residual, fused SwiGLU gate/up
2x11008x4096, down-proj 4096x11008 + residual): four launches through the C
ABI.  Steps cycle through the 32 distinct layers of a random-init 7B model
(3.36 GB of int4 weights), so every step streams its 105 MB from HBM and not
from the 256 MB Infinity Cache.  Launches are replayed from a captured
hipGraph so the host's per-call cost never bounds what the GPU does.

Prints ONE JSON line: whole-job HBM GB/s over the algorithmic bytes of the
mat-vec set (`value`), the roofline record of the dominant kernel (fused
SwiGLU), the single 4096x4096 mat-vec (configs[0]) and the 13B layer set
(configs[2]), decode attention GB/s at 512/2048/4096 rows, full greedy decode
tokens/s (128-token prompt + 256 generated tokens), and the reference's
single-threaded C# CPU path (restated in C) timed beside it.

Every timed figure comes from at least 100 graph replays after warm-up (HIP
events on the library's stream), with the spread (p10 / median / p90) over at
least 50 replays timed one by one; `steps` is what was really timed.
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# HBM bytes per launch of the dominant kernel (fused SwiGLU, 46 880 256 algorithmic bytes), measured with
# two rocprofv3 --pmc runs of `bench.py --only kernel,calib` (counters cannot be read from inside this
# process): (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000) x 1024.  The figure belongs to one state of the
# kernel's source: when csrc/int4_kernels.hpp no longer hashes to the value below, the kernel has changed
# since the counters were read and `roofline.traffic` is reported as null until they are read again.
SWIGLU_HBM_TRAFFIC_BYTES = 47048947
SWIGLU_HBM_TRAFFIC_SOURCE_SHA16 = "c7112bb214b4b729"
MIN_REPLAYS = 100   # graph replays behind every headline figure
MIN_SAMPLES = 50    # replays timed one by one for the spread
HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Events:
    def __init__(self, capi):
        self.capi = capi
        self.a, self.b = C.c_void_p(), C.c_void_p()
        capi.call("llama2_event_create", C.byref(self.a))
        capi.call("llama2_event_create", C.byref(self.b))

    def start(self):
        self.capi.call("llama2_event_record", self.a)

    def stop_ms(self):
        self.capi.call("llama2_event_record", self.b)
        ms = C.c_float()
        self.capi.call("llama2_event_elapsed_ms", self.a, self.b, C.byref(ms))
        return float(ms.value)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3200)
    ap.add_argument("--warmup", type=int, default=320)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--only", default="", help="comma list of legs: set,kernel,cfg0,cfg2,calib,attn,chain,decode,sampler,repack,cpu "
                                               "(default: all but calib)")
    ap.add_argument("--eager", action="store_true",
                    help="issue every launch directly instead of replaying captured graphs.  For runs under rocprofv3, "
                         "whose kernel tracing has crashed the profiled process inside hipGraphLaunch (now and then, on "
                         "graphs of any size): the trace's per-kernel durations do not depend on how a launch was issued; "
                         "the bench's own event timings then include the host's launch gaps and are not the ones to quote")
    ap.add_argument("--decode-mode", default="fused_graph",
                    choices=["modules", "fused", "fused_graph", "persistent", "persistent_graph"])
    args = ap.parse_args()
    if args.eager:  # no captured graph anywhere in the process, the decoder's included
        args.decode_mode = {"fused_graph": "fused", "persistent_graph": "persistent"}.get(args.decode_mode, args.decode_mode)
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU (batch-1 decode has no cross-GPU exchange to measure); "
            "--gpus %d is not supported" % args.gpus)
        sys.exit(2)
    legs = set(args.only.split(",")) if args.only else {"set", "kernel", "cfg0", "cfg2", "attn", "chain", "decode", "sampler",
                                                        "repack", "cpu"}

    from managedllama2_amd import capi, synth
    from managedllama2_amd.device import DeviceVariable, init
    from managedllama2_amd.transformer import Transformer

    init(0)
    cfg = dict(synth.LLAMA2_7B)  # seq_len 4096: room for the attention leg
    dim, hidden, n_layers = cfg["dim"], cfg["hidden_dim"], cfg["n_layers"]
    sizes = synth.layer_matvec_set_bytes(dim, hidden)
    zs, ss, ws = (lambda t: (t[2], t[1], t[0]))(synth.qweight_sizes(dim))
    hzs, hss, hws = (lambda t: (t[2], t[1], t[0]))(synth.qweight_sizes(hidden))

    # ---- the random-init 7B model (configs[4] distributions), generated layer by layer
    t0 = time.time()
    rng = synth.rng_for(1, 7)
    first_layer = []

    def lazy_layers():
        for l in range(n_layers):
            hl = synth.random_layer(rng, dim, hidden)
            if l == 0:
                first_layer.append(hl)  # kept on the host for the CPU baseline
            yield hl

    host = {"embedding": synth.normal_f16(rng, cfg["vocab_size"] * dim, 0.02),
            "classifier": synth.normal_f16(rng, cfg["vocab_size"] * dim, 0.02),
            "rms_final": np.ones(dim, np.float16), "layers": lazy_layers()}
    mode = {"modules": capi.DECODE_MODULES, "fused": capi.DECODE_FUSED,
            "fused_graph": capi.DECODE_FUSED | capi.DECODE_GRAPH,
            "persistent": capi.DECODE_FUSED | capi.DECODE_PERSISTENT,
            "persistent_graph": capi.DECODE_FUSED | capi.DECODE_PERSISTENT | capi.DECODE_GRAPH}[args.decode_mode]
    model = Transformer(cfg, host, mode=mode)
    del host
    layers = model.weights.layers
    log("generated + uploaded the 7B model (%.2f GB of int4 layers) in %.1f s" %
        (n_layers * (sizes["total"] - 126_000) / 1e9, time.time() - t0))

    xb_host = synth.normal_f16(rng, dim)
    xb = DeviceVariable.from_host(xb_host)
    x = DeviceVariable.zeros(np.float16, dim)
    q = DeviceVariable.zeros(np.float16, dim)
    kc = DeviceVariable.zeros(np.float16, dim)
    vc = DeviceVariable.zeros(np.float16, dim)
    h = DeviceVariable.zeros(np.float16, hidden)

    def qkv(L):
        capi.call("llama2_qkv_mat_vec", q.ptr, kc.ptr, vc.ptr, xb.ptr,
                  L.queryWeight.Weight.ptr, L.queryWeight.Zeros.ptr, L.queryWeight.Scales.ptr,
                  L.keyWeight.Weight.ptr, L.keyWeight.Zeros.ptr, L.keyWeight.Scales.ptr,
                  L.valueWeight.Weight.ptr, L.valueWeight.Zeros.ptr, L.valueWeight.Scales.ptr,
                  dim, dim, zs, ss, ws)

    def oproj(L):
        w = L.outputWeight
        capi.call("llama2_mat_vec_residual_int4", x.ptr, xb.ptr, w.Weight.ptr, w.Zeros.ptr, w.Scales.ptr,
                  dim, dim, zs, ss, ws)

    def swiglu(L):
        g, u = L.gateWeight, L.upWeight
        capi.call("llama2_mat_vec_swiglu", h.ptr, xb.ptr, g.Weight.ptr, g.Zeros.ptr, g.Scales.ptr,
                  u.Weight.ptr, u.Zeros.ptr, u.Scales.ptr, dim, hidden, zs, ss, ws)

    def down(L):
        w = L.downWeight
        capi.call("llama2_mat_vec_residual_int4", x.ptr, h.ptr, w.Weight.ptr, w.Zeros.ptr, w.Scales.ptr,
                  hidden, dim, hzs, hss, hws)

    def step(i):
        L = layers[i % n_layers]
        qkv(L)
        oproj(L)
        swiglu(L)
        down(L)

    ev = Events(capi)

    class Eager:
        def __init__(self, fn, n):
            self.fn, self.n = fn, n

    def destroy(graph):
        for g in (graph if isinstance(graph, list) else [graph]):
            if not isinstance(g, Eager):
                capi.call("llama2_graph_destroy", g)

    def capture(fn, n):
        """Record n calls of fn(i) into one hipGraph (--eager: remember them, to be issued one by one)."""
        if args.eager:
            return Eager(fn, n)
        g = C.c_void_p()
        capi.call("llama2_graph_begin_capture")
        for i in range(n):
            fn(i)
        capi.call("llama2_graph_end_capture", C.byref(g))
        return g

    def launch(graph):
        """One replay (`graph` may be a list of graphs that together make up the replay)."""
        for g in (graph if isinstance(graph, list) else [graph]):
            if isinstance(g, Eager):
                for i in range(g.n):
                    g.fn(i)
            else:
                capi.call("llama2_graph_launch", g)

    def timed_replays(graph, replays):
        capi.call("llama2_sync")
        ev.start()
        for _ in range(replays):
            launch(graph)
        ms = ev.stop_ms()
        capi.call("llama2_sync")
        return ms

    def measure(graph, units_per_replay, replays=MIN_REPLAYS, warmup=3):
        """Mean microseconds per unit over `replays` (>= MIN_REPLAYS) back-to-back replays, and the
        p10 / median / p90 over MIN_SAMPLES replays timed one by one."""
        replays = max(replays, MIN_REPLAYS)
        for _ in range(max(warmup, 1)):
            launch(graph)
        us = 1e3 * timed_replays(graph, replays) / (replays * units_per_replay)
        one_by_one = []
        for _ in range(MIN_SAMPLES):
            ev.start()
            launch(graph)
            one_by_one.append(1e3 * ev.stop_ms() / units_per_replay)
        spread = [round(float(v), 3) for v in np.percentile(np.array(one_by_one), [10, 50, 90])]
        return us, spread, replays

    result = {
        "metric": "int4 mat-vec HBM GB/s, Llama-2-7B decoder-layer mat-vec set, batch 1",
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights x f16 activations, f32 accumulate", "data": "synthetic",
        "config": {"workload": "configs[1]: 7B layer mat-vec set (QKV, o+res, SwiGLU, down+res), "
                               "%d distinct layers cycled (cold HBM)" % n_layers,
                   "dim": dim, "hidden_dim": hidden, "algorithmic_bytes_per_step": sizes["total"]},
    }

    if "set" in legs:
        # one graph = one pass over all distinct layers; K steps = K / n_layers replays, at least MIN_REPLAYS
        graph = capture(step, n_layers)  # 4 launches x 32 layers in one graph
        wall0 = time.perf_counter()
        us, spread, replays = measure(graph, n_layers, replays=-(-args.steps // n_layers),
                                      warmup=max(args.warmup // n_layers, 1))
        wall = time.perf_counter() - wall0
        destroy(graph)
        steps = replays * n_layers
        ms_per_step = us * 1e-3
        gbps = sizes["total"] / (ms_per_step * 1e-3) / 1e9
        result.update(steps=steps, steps_requested=args.steps, replays=replays, value=round(gbps, 1),
                      ms_per_step=round(ms_per_step, 5), pct_of_hbm_peak=round(100 * gbps / HBM_PEAK_GBPS, 2),
                      wall_ms_per_step_incl_spread_runs=round(1e3 * wall / (steps + MIN_SAMPLES * n_layers), 5),
                      us_per_step_p10_median_p90=spread, spread_samples=MIN_SAMPLES)
        log("layer mat-vec set: %.2f us/step over %d replays (p10 %.2f / median %.2f / p90 %.2f), %.0f GB/s (%.1f%% of 8 TB/s)" %
            (us, replays, spread[0], spread[1], spread[2], gbps, 100 * gbps / HBM_PEAK_GBPS))

    if "kernel" in legs:
        per_kernel = {}
        for name, fn in (("qkv", qkv), ("o", oproj), ("swiglu", swiglu), ("down", down)):
            graph = capture(lambda i, fn=fn: fn(layers[i % n_layers]), n_layers)
            us, spread, replays = measure(graph, n_layers)
            destroy(graph)
            per_kernel[name] = {"us": round(us, 3), "us_p10_median_p90": spread, "launches": replays * n_layers,
                                "GBps": round(sizes[name] / us / 1e3, 1), "bytes": sizes[name],
                                "frac_of_hbm_peak": round(sizes[name] / us / 1e3 / HBM_PEAK_GBPS, 4)}
            log("  %-7s %8.2f us  %7.0f GB/s  (%d B)" % (name, us, sizes[name] / us / 1e3, sizes[name]))
        dom = per_kernel["swiglu"]
        import hashlib
        src = os.path.join(ROOT, "managedllama2_amd", "csrc", "int4_kernels.hpp")
        sha16 = hashlib.sha256(open(src, "rb").read()).hexdigest()[:16] if os.path.exists(src) else None
        fresh = sha16 == SWIGLU_HBM_TRAFFIC_SOURCE_SHA16
        result["roofline"] = {"bound": "hbm", "kernel": "int4_matvec_span_kernel<2, SWIGLU, STAGE_X, 2, 8, 3> (fused gate/up, 2x11008x4096)",
                              "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                              "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4),
                              "traffic": SWIGLU_HBM_TRAFFIC_BYTES if fresh else None,
                              "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --only kernel,calib`, "
                                                "scaled by a 1 GiB copy kernel (factors 2.000 / 1.000): profiles/"
                                                "int4_matvec_7b_layer_set_hbm_traffic.md; read for the kernel source "
                                                "with sha256[:16] = %s, this run's source: %s%s" %
                                                (SWIGLU_HBM_TRAFFIC_SOURCE_SHA16, sha16,
                                                 "" if fresh else " (changed since: counters not re-read, traffic withheld)"),
                              "algorithmic_bytes_per_launch": dom["bytes"], "avg_launch_us": dom["us"],
                              "launches_timed": dom["launches"]}
        result["per_kernel"] = per_kernel

    if "cfg0" in legs:
        # configs[0]: ONE int4 mat-vec 4096 x 4096 (plain, and with the residual epilogue), cycled over the
        # model's 128 distinct q / k / v / o tensors (1.1 GB: cold HBM).  8 732 672 algorithmic bytes
        # (+ 8 192 for the residual read); floor at 8 TB/s: 1.09 us.
        tensors = [w for L in layers for w in (L.queryWeight, L.keyWeight, L.valueWeight, L.outputWeight)]
        b0 = synth.qweight_bytes(dim, dim) + 2 * dim + 2 * dim
        cfg0 = {}
        for name, entry, nbytes in (("plain", "llama2_mat_vec_int4", b0), ("residual", "llama2_mat_vec_residual_int4", b0 + 2 * dim)):
            graphs = capture(lambda i, entry=entry: capi.call(entry, x.ptr, xb.ptr, tensors[i].Weight.ptr,
                                                               tensors[i].Zeros.ptr, tensors[i].Scales.ptr,
                                                               dim, dim, zs, ss, ws), len(tensors))
            us, spread, replays = measure(graphs, len(tensors))
            destroy(graphs)
            cfg0[name] = {"us": round(us, 3), "us_p10_median_p90": spread, "launches": replays * len(tensors), "bytes": nbytes,
                          "GBps": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                          "floor_us_at_8TBps": round(nbytes / 8e6, 3)}
            log("  cfg0 %-9s %6.2f us  %6.0f GB/s (%.1f%% of peak; floor %.2f us)" %
                (name, us, nbytes / us / 1e3, 100 * nbytes / us / 1e3 / HBM_PEAK_GBPS, nbytes / 8e6))
        cfg0["workload"] = "configs[0]: single AWQ int4 mat-vec K = N = 4096, %d distinct tensors cycled" % len(tensors)
        result["cfg0"] = cfg0

    if "cfg2" in legs:
        # configs[2]: the Llama-2-13B layer mat-vec set (dim 5120, hidden 13824; 14 padded zero words per
        # down-proj row) over 4 distinct layers (660 MB: cold HBM).  164 960 256 algorithmic bytes; floor 20.6 us.
        d13, h13, n13 = synth.LLAMA2_13B["dim"], synth.LLAMA2_13B["hidden_dim"], 4
        s13 = synth.layer_matvec_set_bytes(d13, h13)
        z13, q13, w13 = (lambda t: (t[2], t[1], t[0]))(synth.qweight_sizes(d13))
        hz13, hq13, hw13 = (lambda t: (t[2], t[1], t[0]))(synth.qweight_sizes(h13))
        from managedllama2_amd.device import QWeight
        rng13 = synth.rng_for(2, 13)
        L13 = []
        for _ in range(n13):
            hl = synth.random_layer(rng13, d13, h13)
            L13.append({k: QWeight.from_host(*hl[k]) for k in ("q", "k", "v", "o", "gate", "up", "down")})
        xb13 = DeviceVariable.from_host(synth.normal_f16(rng13, d13))
        x13, q13v, k13v, v13v = (DeviceVariable.zeros(np.float16, d13) for _ in range(4))
        hbuf13 = DeviceVariable.zeros(np.float16, h13)

        def p3(w):
            return (w.Weight.ptr, w.Zeros.ptr, w.Scales.ptr)

        def qkv13(L):
            capi.call("llama2_qkv_mat_vec", q13v.ptr, k13v.ptr, v13v.ptr, xb13.ptr, *p3(L["q"]), *p3(L["k"]), *p3(L["v"]),
                      d13, d13, z13, q13, w13)

        def o13(L):
            capi.call("llama2_mat_vec_residual_int4", x13.ptr, xb13.ptr, *p3(L["o"]), d13, d13, z13, q13, w13)

        def sw13(L):
            capi.call("llama2_mat_vec_swiglu", hbuf13.ptr, xb13.ptr, *p3(L["gate"]), *p3(L["up"]), d13, h13, z13, q13, w13)

        def dn13(L):
            capi.call("llama2_mat_vec_residual_int4", x13.ptr, hbuf13.ptr, *p3(L["down"]), h13, d13, hz13, hq13, hw13)

        cfg2 = {"workload": "configs[2]: 13B layer mat-vec set, %d distinct layers cycled" % n13,
                "algorithmic_bytes_per_step": s13["total"], "floor_us_at_8TBps": round(s13["total"] / 8e6, 2)}
        graph = capture(lambda i: [f(L13[i % n13]) for f in (qkv13, o13, sw13, dn13)], n13)
        us, spread, replays = measure(graph, n13, replays=4 * MIN_REPLAYS)
        destroy(graph)
        cfg2["set"] = {"us": round(us, 3), "us_p10_median_p90": spread, "steps": replays * n13,
                       "GBps": round(s13["total"] / us / 1e3, 1),
                       "frac_of_hbm_peak": round(s13["total"] / us / 1e3 / HBM_PEAK_GBPS, 4)}
        log("  cfg2 13B layer set %6.2f us  %6.0f GB/s (%.1f%% of peak; floor %.1f us)" %
            (us, s13["total"] / us / 1e3, 100 * s13["total"] / us / 1e3 / HBM_PEAK_GBPS, s13["total"] / 8e6))
        for name, fn in (("qkv", qkv13), ("o", o13), ("swiglu", sw13), ("down", dn13)):
            graph = capture(lambda i, fn=fn: fn(L13[i % n13]), n13)
            us, spread, replays = measure(graph, n13, replays=4 * MIN_REPLAYS)
            destroy(graph)
            cfg2[name] = {"us": round(us, 3), "us_p10_median_p90": spread, "bytes": s13[name],
                          "GBps": round(s13[name] / us / 1e3, 1),
                          "frac_of_hbm_peak": round(s13[name] / us / 1e3 / HBM_PEAK_GBPS, 4)}
            log("    13B %-7s %8.2f us  %7.0f GB/s" % (name, us, s13[name] / us / 1e3))
        result["cfg2"] = cfg2
        for L in L13:
            for w in L.values():
                for b in (w.Weight, w.Zeros, w.Scales):
                    b.free()

    if "calib" in legs:
        # a plain copy of known size: what FETCH_SIZE / WRITE_SIZE read for it scales the counters
        # of the mat-vec kernels (rocprofv3 --pmc runs, see profiles/)
        n = 1 << 30
        src, dst = DeviceVariable.zeros(np.uint8, n), DeviceVariable.zeros(np.uint8, n)
        capi.call("llama2_sync")
        ev.start()
        for _ in range(4):
            capi.call("llama2_memcpy_d2d", dst.ptr, src.ptr, n)
        ms = ev.stop_ms() / 4
        result["copy_calibration"] = {"bytes_read": n, "bytes_written": n, "us": round(1e3 * ms, 1),
                                      "GBps_read_plus_write": round(2 * n / ms / 1e6, 1)}
        log("copy calibration: 1 GiB -> 1 GiB in %.1f us (%.0f GB/s read+write)" % (1e3 * ms, 2 * n / ms / 1e6))
        src.free()
        dst.free()

    if "attn" in legs:
        # configs[3]: decode attention over the fp16 KV cache, 32 heads x 128, RoPE at pos = S on the
        # newest row, scores, softmax, weighted value sum; cycled over the 32 layers' cache slices
        rs = model.runstate
        seq_cap = model.config.seq_len
        kv_bytes = rs.keyCache.nbytes
        fill = synth.normal_f16(synth.rng_for(3), 1 << 22)
        for off in range(0, kv_bytes // 2, fill.size):  # N(0,1) values everywhere
            n = min(fill.size, kv_bytes // 2 - off)
            rs.keyCache.copy_to_device(fill[:n], off)
            rs.valueCache.copy_to_device(fill[:n], off)
        rs.q.copy_to_device(synth.normal_f16(synth.rng_for(4), dim))
        hs, heads = dim // cfg["n_heads"], cfg["n_heads"]
        scale = 1.0 / math.sqrt(hs)
        attn = {}
        for S in (512, 2048, 4096):
            if S > seq_cap:
                continue
            nbytes = 2 * S * dim * 2 + 2 * dim * 2

            def modules(i, S=S):
                lo = (i % n_layers) * seq_cap * dim
                capi.call("llama2_rope", rs.q.ptr, rs.keyCache.offset_pointer(lo + (S - 1) * dim), heads, hs, S,
                          10000.0, heads)
                capi.call("llama2_mat_vec_strided", rs.attention.ptr, rs.q.ptr, rs.keyCache.offset_pointer(lo),
                          hs, S, hs, hs, dim, S, scale, heads)
                capi.call("llama2_softmax", rs.attention.ptr, S, heads)
                capi.call("llama2_vec_mat", rs.xb.ptr, rs.attention.ptr, rs.valueCache.offset_pointer(lo),
                          hs, S, hs, hs, dim, heads)

            def fused(i, S=S):
                lo = (i % n_layers) * seq_cap * dim
                capi.call("llama2_rope", rs.q.ptr, rs.keyCache.offset_pointer(lo + (S - 1) * dim), heads, hs, S,
                          10000.0, heads)
                capi.call("llama2_multi_head_attention", rs.xb.ptr, rs.q.ptr, rs.keyCache.offset_pointer(lo),
                          rs.valueCache.offset_pointer(lo), hs, dim, S, scale, heads)

            def one_launch(i, S=S):
                lo = (i % n_layers) * seq_cap * dim
                capi.call("llama2_rope_multi_head_attention", rs.xb.ptr, rs.q.ptr, rs.keyCache.offset_pointer(lo),
                          rs.valueCache.offset_pointer(lo), hs, dim, S, scale, heads, S, 10000.0)

            row = {"bytes": nbytes}
            for name, fn in (("modules", modules), ("fused", fused), ("one_launch", one_launch)):
                fn(0)  # sizes the library's scratch before capture
                graph = capture(fn, n_layers)
                us, spread, replays = measure(graph, n_layers)
                destroy(graph)
                row[name] = {"us": round(us, 2), "us_p10_median_p90": spread, "launches": replays * n_layers,
                             "GBps": round(nbytes / us / 1e3, 1)}
            attn["S=%d" % S] = row
            log("  attention S=%-5d rope+scores+softmax+vecmat %7.2f us %6.0f GB/s | rope+fused %7.2f us %6.0f GB/s | "
                "one launch %7.2f us %6.0f GB/s" %
                (S, row["modules"]["us"], row["modules"]["GBps"], row["fused"]["us"], row["fused"]["GBps"],
                 row["one_launch"]["us"], row["one_launch"]["GBps"]))
        result["attention"] = attn

    if "chain" in legs:
        # The whole-step persistent kernel (one launch per token, vectors handed over between workgroups as
        # tagged words) on the same weights: its mat-vec chain (32 layers, attention skipped) per layer, and
        # the full greedy decode through it.  Reported beside the launch sequence; the faster one is the default.
        dec = C.c_void_p()
        pmode = capi.DECODE_FUSED | capi.DECODE_PERSISTENT | capi.DECODE_GRAPH
        capi.call("llama2_decode_create", C.byref(dec), C.byref(model.config), C.byref(model._w_struct),
                  C.byref(model._s_struct), pmode)
        graph = capture(lambda i: capi.call("llama2_decode_matvec_chain", dec, xb.ptr, x.ptr), 1)
        us, spread, replays = measure(graph, n_layers)
        destroy(graph)
        capi.call("llama2_decode_check", dec)
        n_prompt, n_gen = 128, 256
        steps = n_prompt + n_gen - 1
        prompt = synth.rng_for(5).integers(3, cfg["vocab_size"], n_prompt).astype(np.int32)
        model.runstate.tokens.copy_to_device(prompt)
        capi.call("llama2_decode_run", dec, 0, 16, n_prompt)
        capi.call("llama2_sync")
        ev.start()
        capi.call("llama2_decode_run", dec, 0, steps, n_prompt)
        ms = ev.stop_ms()
        capi.call("llama2_decode_check", dec)
        ptoks = model.runstate.tokens.to_host(n_prompt + n_gen)
        result["persistent_step"] = {"matvec_chain_us_per_layer": round(us, 3), "us_p10_median_p90": spread,
                                     "chain_launches": replays, "GBps": round(sizes["total"] / us / 1e3, 1),
                                     "decode_tokens_per_s": round(steps / (ms * 1e-3), 1),
                                     "last_tokens": [int(t) for t in ptoks[-4:]]}
        log("persistent step: mat-vec chain %.2f us/layer (%.0f GB/s), decode %.1f tok/s" %
            (us, sizes["total"] / us / 1e3, steps / (ms * 1e-3)))
        capi.call("llama2_decode_destroy", dec)

    if "decode" in legs:
        # configs[4]: 128 seeded prompt tokens, 256 greedy tokens, every step on the device
        n_prompt, n_gen = 128, 256
        steps = n_prompt + n_gen - 1
        prompt = synth.rng_for(5).integers(3, cfg["vocab_size"], n_prompt).astype(np.int32)
        model.runstate.tokens.copy_to_device(prompt)
        capi.call("llama2_decode_run", model._decoder, 0, 16, n_prompt)  # warm-up
        capi.call("llama2_sync")
        ev.start()
        capi.call("llama2_decode_run", model._decoder, 0, steps, n_prompt)
        ms = ev.stop_ms()
        toks = model.runstate.tokens.to_host(n_prompt + n_gen)
        tok_s = steps / (ms * 1e-3)
        kv_avg = 2 * n_layers * (steps + 1) / 2 * dim * 2
        bytes_tok = (n_layers * (sizes["total"] - 126_000 + 2 * 2 * dim) + 2 * cfg["vocab_size"] * dim
                     + 2 * dim + 2 * dim + kv_avg)
        result["decode"] = {"tokens_per_s": round(tok_s, 1), "ms_per_token": round(ms / steps, 4),
                            "forward_steps": steps, "prompt": n_prompt, "generated": n_gen,
                            "mode": args.decode_mode,
                            "GBps": round(bytes_tok * tok_s / 1e9, 1),
                            "pct_of_hbm_peak": round(100 * bytes_tok * tok_s / 1e9 / HBM_PEAK_GBPS, 2),
                            "bandwidth_bound_tokens_per_s": round(HBM_PEAK_GBPS * 1e9 / bytes_tok, 1),
                            "last_tokens": [int(t) for t in toks[-4:]]}
        # the same loop late in the context: 64 steps from position 3968 of 4096 (attention reads ~2 x 1 GB of cache)
        far = cfg["seq_len"] - 128
        capi.call("llama2_decode_run", model._decoder, far, 8, 0)
        capi.call("llama2_sync")
        ev.start()
        capi.call("llama2_decode_run", model._decoder, far, 64, 0)
        far_ms = ev.stop_ms()
        result["decode"]["tokens_per_s_at_position_%d" % far] = round(64 / (far_ms * 1e-3), 1)
        log("decode at positions %d..%d: %.1f tok/s" % (far, far + 63, 64 / (far_ms * 1e-3)))
        # the reference's own loop shape (Transformer.Generate: forward every step, sample and read the token
        # back on the host for every generated token) over the same positions and launches: what a host that
        # keeps its loop gets
        t1 = time.perf_counter()
        n_host = sum(1 for _ in model.Generate(prompt, steps, stop_on_special=False))
        host_tok_s = n_host / (time.perf_counter() - t1)
        result["decode"]["host_loop_tokens_per_s"] = round(host_tok_s, 1)
        log("decode, host loop with one read-back per token: %.1f tok/s" % host_tok_s)
        log("decode: %.1f tok/s (%.3f ms/token, %.0f GB/s = %.1f%% of peak; ceiling %.0f tok/s)" %
            (tok_s, ms / steps, bytes_tok * tok_s / 1e9, 100 * bytes_tok * tok_s / 1e9 / HBM_PEAK_GBPS,
             HBM_PEAK_GBPS * 1e9 / bytes_tok))

    if "sampler" in legs:
        # Sampler.Sample with the reference's defaults (temperature 0.5, top-p 0.9) on 32000 logits:
        # the four module launches, the one-launch sampler, and the device-resident decode loop with it
        vocab = cfg["vocab_size"]
        logits_host = synth.normal_f16(synth.rng_for(6), vocab, 2.0)
        lg, idx = DeviceVariable.from_host(logits_host), DeviceVariable.zeros(np.int32, vocab)
        src = DeviceVariable.from_host(logits_host)
        tok = DeviceVariable.zeros(np.int32, 2)
        temp, top_p = 0.5, 0.9
        sampler = {}

        def timed(name, fn):
            graph = capture(lambda i: (capi.call("llama2_memcpy_d2d", lg.ptr, src.ptr, vocab * 2), fn()), 16)
            base = capture(lambda i: capi.call("llama2_memcpy_d2d", lg.ptr, src.ptr, vocab * 2), 16)
            for g in (graph, base):
                launch(g)
            us = 1e3 * (timed_replays(graph, 20) - timed_replays(base, 20)) / (20 * 16)
            destroy(graph)
            destroy(base)
            sampler[name] = round(us, 2)

        timed("softmax_logits_us", lambda: capi.call("llama2_softmax_logits", lg.ptr, vocab, temp, idx.ptr))
        timed("sort_us", lambda: capi.call("llama2_sort", lg.ptr, idx.ptr, vocab))
        timed("cumulative_sum_us", lambda: capi.call("llama2_cumulative_sum", lg.ptr, vocab))
        timed("sample_top_p_us", lambda: capi.call("llama2_sample_top_p", lg.ptr, idx.ptr, vocab, 0.45, tok.ptr, 1))
        timed("four_modules_us", lambda: (capi.call("llama2_softmax_logits", lg.ptr, vocab, temp, idx.ptr),
                                          capi.call("llama2_sort", lg.ptr, idx.ptr, vocab),
                                          capi.call("llama2_cumulative_sum", lg.ptr, vocab),
                                          capi.call("llama2_sample_top_p", lg.ptr, idx.ptr, vocab, 0.45, tok.ptr, 1)))
        timed("one_launch_us", lambda: capi.call("llama2_sample", lg.ptr, idx.ptr, vocab, temp, top_p, 0.5, tok.ptr, 1))
        n_prompt, n_gen = 128, 256
        steps = n_prompt + n_gen - 1
        prompt = synth.rng_for(5).integers(3, vocab, n_prompt).astype(np.int32)
        model.runstate.tokens.copy_to_device(prompt)
        capi.call("llama2_decode_run_sampled", model._decoder, 0, 16, n_prompt, temp, top_p, 1)  # warm-up
        capi.call("llama2_sync")
        ev.start()
        capi.call("llama2_decode_run_sampled", model._decoder, 0, steps, n_prompt, temp, top_p, 1)
        ms = ev.stop_ms()
        sampler["decode_tokens_per_s"] = round(steps / (ms * 1e-3), 1)
        sampler["decode_ms_per_token"] = round(ms / steps, 4)
        sampler["temperature"], sampler["top_p"] = temp, top_p
        # the reference's loop shape with its sampler: forward, llama2_decode_sample_top_p, token read back per step
        if model._decoder is not None:
            sp, coins = model.sampler, np.random.default_rng(7)
            sp.temperature, sp.topP, sp.random = temp, top_p, coins.random
            t1 = time.perf_counter()
            n_host = sum(1 for _ in model.Generate(prompt, steps, stop_on_special=False))
            sampler["host_loop_tokens_per_s"] = round(n_host / (time.perf_counter() - t1), 1)
            sp.temperature = 0.0
        result["sampler"] = sampler
        log("sampler (32000 logits, T=0.5, top-p 0.9): softmax %.1f + sort %.1f + cumsum %.1f + pick %.1f us; "
            "4 launches %.1f us, one launch %.1f us; sampled decode %.1f tok/s (host loop %s)" %
            (sampler["softmax_logits_us"], sampler["sort_us"], sampler["cumulative_sum_us"],
             sampler["sample_top_p_us"], sampler["four_modules_us"], sampler["one_launch_us"],
             sampler["decode_tokens_per_s"], sampler.get("host_loop_tokens_per_s")))

    if "repack" in legs:
        # the converter's repack of the 7B weight tensors (AWQ GEMM words -> output-major words):
        # every word read once and written once
        repack = {}
        for name, (K, N) in (("qkvo_4096x4096", (dim, dim)), ("gate_up_4096x11008", (dim, hidden)),
                             ("down_11008x4096", (hidden, dim))):
            words = K * N // 8
            src_w = DeviceVariable.from_host(synth.rng_for(8, K, N).integers(0, 2 ** 32, words, dtype=np.uint64)
                                             .astype(np.uint32))
            dst_w = DeviceVariable(np.uint32, words)
            capi.call("llama2_repack_qdata", dst_w.ptr, src_w.ptr, K, N)
            capi.call("llama2_sync")
            ev.start()
            for _ in range(20):
                capi.call("llama2_repack_qdata", dst_w.ptr, src_w.ptr, K, N)
            us = 1e3 * ev.stop_ms() / 20
            repack[name] = {"us": round(us, 2), "GBps_read_plus_write": round(2 * words * 4 / us / 1e3, 1)}
            src_w.free()
            dst_w.free()
        result["repack"] = repack
        log("repack (read+write): " + ", ".join("%s %.1f us %.0f GB/s" % (k, v["us"], v["GBps_read_plus_write"])
                                                for k, v in repack.items()))

    if "cpu" in legs and args.cpu_seconds > 0:
        from oracle import oracle
        hm_layer = first_layer[0]
        lp = oracle.LayerPtr()
        for name in ("q", "k", "v", "o", "gate", "up", "down"):
            W, Z, S = hm_layer[name]
            setattr(lp, name, oracle.QWeightPtr(oracle._u(W), oracle._u(Z), oracle._h(S)))
        oracle.set_threads(1)
        x0 = np.zeros(dim, np.float16)
        n_sets, spent = 0, 0.0
        while spent < args.cpu_seconds and n_sets < 64:
            t1 = time.perf_counter()
            oracle.ref_layer_matvec_set(lp, dim, hidden, xb_host, x0)
            spent += time.perf_counter() - t1
            n_sets += 1
        cpu_gbps = sizes["total"] * n_sets / spent / 1e9
        result["cpu_baseline"] = {"value": round(cpu_gbps, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                                  "sample": "%d x the same 7B layer mat-vec set (HostQWeight.Unpack + fp32 "
                                            "sequential dot, as the reference's C# tests), %.1f s" % (n_sets, spent),
                                  "seconds_per_step": round(spent / n_sets, 3), "host_cpus": os.cpu_count()}
        log("cpu baseline: %.3f s per layer set on 1 core (%.4f GB/s)" % (spent / n_sets, cpu_gbps))

    model.close()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
