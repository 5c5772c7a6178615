#!/usr/bin/env python3
"""Benchmark of the quantized batch-1 decode hot path on one MI355X.

A "step" is one Llama-2-7B decoder layer's int4 mat-vec set at batch 1 (fused
QKV 3x4096x4096, o-proj 4096x4096 + residual, fused SwiGLU gate/up
2x11008x4096, down-proj 4096x11008 + residual): four launches through the C
ABI.  Steps cycle through 32 distinct layers of weights (3.36 GB), so every
step streams its 105 MB from HBM and not from the 256 MB Infinity Cache.

Prints ONE JSON line: whole-job HBM GB/s over the algorithmic bytes of the
mat-vec set, the roofline record of the dominant kernel (fused SwiGLU), and
the reference's single-threaded C# CPU path (restated in C) timed beside it.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

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
    ap.add_argument("--layers", type=int, default=32, help="distinct weight copies cycled through")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--only", default="", help="comma list of legs to run: set,kernel,cpu (default all)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU (batch-1 decode has no cross-GPU exchange to measure); "
            "--gpus %d is not supported" % args.gpus)
        sys.exit(2)
    legs = set(args.only.split(",")) if args.only else {"set", "kernel", "cpu"}

    from managedllama2_amd import capi, synth
    from managedllama2_amd.device import DeviceVariable, QWeight, init

    init(0)
    dim, hidden = 4096, 11008
    sizes = synth.layer_matvec_set_bytes(dim, hidden)
    zs, ss, ws = (lambda t: (t[2], t[1], t[0]))(synth.qweight_sizes(dim))
    hzs, hss, hws = (lambda t: (t[2], t[1], t[0]))(synth.qweight_sizes(hidden))

    t0 = time.time()
    rng = synth.rng_for(1, 7)
    host_layers = []
    layers = []
    for l in range(args.layers):
        hl = synth.random_layer(rng, dim, hidden)
        if l == 0:
            host_layers.append(hl)  # kept for the CPU baseline
        layers.append({k: QWeight.from_host(*hl[k]) for k in ("q", "k", "v", "o", "gate", "up", "down")})
    log("generated + uploaded %d layers (%.2f GB) in %.1f s" %
        (args.layers, args.layers * (sizes["total"] - 126_000) / 1e9, time.time() - t0))

    xb_host = synth.normal_f16(rng, dim)
    xb = DeviceVariable.from_host(xb_host)
    x = DeviceVariable.zeros(np.float16, dim)
    q = DeviceVariable.zeros(np.float16, dim)
    kc = DeviceVariable.zeros(np.float16, dim)
    vc = DeviceVariable.zeros(np.float16, dim)
    h = DeviceVariable.zeros(np.float16, hidden)

    def qkv(L):
        capi.call("llama2_qkv_mat_vec", q.ptr, kc.ptr, vc.ptr, xb.ptr,
                  L["q"].Weight.ptr, L["q"].Zeros.ptr, L["q"].Scales.ptr,
                  L["k"].Weight.ptr, L["k"].Zeros.ptr, L["k"].Scales.ptr,
                  L["v"].Weight.ptr, L["v"].Zeros.ptr, L["v"].Scales.ptr, dim, dim, zs, ss, ws)

    def oproj(L):
        capi.call("llama2_mat_vec_residual_int4", x.ptr, xb.ptr, L["o"].Weight.ptr, L["o"].Zeros.ptr,
                  L["o"].Scales.ptr, dim, dim, zs, ss, ws)

    def swiglu(L):
        capi.call("llama2_mat_vec_swiglu", h.ptr, xb.ptr, L["gate"].Weight.ptr, L["gate"].Zeros.ptr,
                  L["gate"].Scales.ptr, L["up"].Weight.ptr, L["up"].Zeros.ptr, L["up"].Scales.ptr,
                  dim, hidden, zs, ss, ws)

    def down(L):
        capi.call("llama2_mat_vec_residual_int4", x.ptr, h.ptr, L["down"].Weight.ptr, L["down"].Zeros.ptr,
                  L["down"].Scales.ptr, hidden, dim, hzs, hss, hws)

    def step(i):
        L = layers[i % len(layers)]
        qkv(L)
        oproj(L)
        swiglu(L)
        down(L)

    ev = Events(capi)

    def capture(fn, n):
        """Record n calls of fn(i) into one hipGraph (one submission per replay,
        so the host's per-call cost never bounds what the GPU is seen to do)."""
        g = C.c_void_p()
        capi.call("llama2_graph_begin_capture")
        for i in range(n):
            fn(i)
        capi.call("llama2_graph_end_capture", C.byref(g))
        return g

    def timed_replays(graph, replays):
        capi.call("llama2_sync")
        ev.start()
        for _ in range(replays):
            capi.call("llama2_graph_launch", graph)
        ms = ev.stop_ms()
        capi.call("llama2_sync")
        return ms
    result = {
        "metric": "int4 mat-vec HBM GB/s, Llama-2-7B decoder-layer mat-vec set, batch 1",
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int4 weights x f16 activations, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "configs[1]: 7B layer mat-vec set (QKV, o+res, SwiGLU, down+res), "
                               "%d distinct weight copies cycled (cold HBM)" % args.layers,
                   "dim": dim, "hidden_dim": hidden, "algorithmic_bytes_per_step": sizes["total"]},
    }

    cycle = len(layers)
    if "set" in legs:
        # one graph = one pass over all distinct layers; K steps = K/cycle replays
        graph = capture(step, cycle)
        replays = max(args.steps // cycle, 1)
        args.steps = replays * cycle
        for _ in range(max(args.warmup // cycle, 1)):
            capi.call("llama2_graph_launch", graph)
        capi.call("llama2_sync")
        wall0 = time.perf_counter()
        ms = timed_replays(graph, replays)
        wall = time.perf_counter() - wall0
        capi.call("llama2_graph_destroy", graph)
        result["steps"] = args.steps
        ms_per_step = ms / args.steps
        gbps = sizes["total"] / (ms_per_step * 1e-3) / 1e9
        result.update(value=round(gbps, 1), ms_per_step=round(ms_per_step, 5),
                      pct_of_hbm_peak=round(100 * gbps / HBM_PEAK_GBPS, 2),
                      wall_ms_per_step=round(1e3 * wall / args.steps, 5))
        log("layer mat-vec set: %.2f us/step, %.0f GB/s (%.1f%% of 8 TB/s)" %
            (1e3 * ms_per_step, gbps, 100 * gbps / HBM_PEAK_GBPS))

    if "kernel" in legs:
        per_kernel = {}
        for name, fn in (("qkv", qkv), ("o", oproj), ("swiglu", swiglu), ("down", down)):
            graph = capture(lambda i, fn=fn: fn(layers[i % cycle]), cycle)
            replays = max(args.steps // cycle // 2, 2)
            capi.call("llama2_graph_launch", graph)
            us = 1e3 * timed_replays(graph, replays) / (replays * cycle)
            capi.call("llama2_graph_destroy", graph)
            per_kernel[name] = {"us": round(us, 3), "GBps": round(sizes[name] / us / 1e3, 1),
                                "bytes": sizes[name]}
            log("  %-7s %8.2f us  %7.0f GB/s  (%d B)" % (name, us, sizes[name] / us / 1e3, sizes[name]))
        dom = per_kernel["swiglu"]
        result["roofline"] = {"bound": "hbm", "kernel": "int4_swiglu_kernel (fused gate/up, 2x11008x4096)",
                              "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                              "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4), "traffic": None,
                              "algorithmic_bytes_per_launch": dom["bytes"], "avg_launch_us": dom["us"]}
        result["per_kernel"] = per_kernel

    if "cpu" in legs and args.cpu_seconds > 0:
        from oracle import oracle
        hm_layer = host_layers[0]
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

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
