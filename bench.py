#!/usr/bin/env python3
"""Benchmark of the quantized-Linear hot path on one MI355X.

Workload (the configuration the metric is quoted on): the seven Linear projections of a Qwen3-4B decoder layer as decode
GEMVs with Q4_0 weights, bf16 activations, M = 1.  One step = one decode token through all 36 layers = 252 GEMV launches
over 2.04 GB of distinct weights (far larger than the 256 MB last-level cache, so every step streams from HBM).
The launches of a step are captured once into a HIP graph and replayed.

Prints ONE JSON line.  `value` is whole-job algorithmic GB/s (weights 18 B per 32-element block + activations + outputs,
divided by wall time of the timed steps, inputs resident in HBM).  `roofline` is the dominant GEMV shape alone
(gate/up projection), timed with HIP events on the launch stream.  `cpu_baseline` times the CPU oracle of the same path on a
bounded sample on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
N_LAYERS = 36


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--wtype", choices=["q4_0", "q8_0"], default="q4_0")
    ap.add_argument("--m", type=int, default=1, help="activation rows of the headline workload (1..8)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the M=4/8 and Q8_0 side measurements")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from mllm_amd import _lib, qlinear as ql, synth

    _lib.check(_lib.lib().mllm_hip_init(0), "mllm_hip_init")
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(synth.SEED_BASE + 1)
    shapes = synth.QWEN3_4B_LAYER
    stream = torch.cuda.current_stream()

    def make_pool(wtype, layers):
        return [{name: ql.PackedQWeight.synthetic(wtype, n, k, gen) for name, (n, k) in shapes.items()}
                for _ in range(layers)]

    def make_io(M):
        xs = {k: torch.randn((M, k), device="cuda", generator=gen).to(torch.bfloat16) for k in (2560, 4096, 9728)}
        ys = {name: torch.empty((M, n), dtype=torch.float32, device="cuda") for name, (n, _) in shapes.items()}
        return xs, ys

    def step_bytes(wtype, M):
        return N_LAYERS * sum(synth.gemv_algorithmic_bytes(wtype, M, n, k, 2) for n, k in shapes.values())

    def run_step(pool, xs, ys):
        for layer in pool:
            for name, w in layer.items():
                ql.linear_q_gemv(w, xs[w.K], None, ql.SCALE_X86_REF, out=ys[name])

    def timed(fn, steps, warmup):
        """warmup, then `steps` calls bracketed by synchronize; returns (wall seconds, HIP-event seconds)"""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(steps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, e0.elapsed_time(e1) * 1e-3

    def graphed(fn):
        if args.no_graph:
            return fn
        fn()  # first launch outside capture (module load, attribute set-up)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g.replay

    def measure_workload(wtype, M, pool, steps, warmup):
        xs, ys = make_io(M)
        replay = graphed(lambda: run_step(pool, xs, ys))
        wall, ev = timed(replay, steps, warmup)
        nbytes = step_bytes(wtype, M)
        return {"GBps": nbytes * steps / wall / 1e9, "ms_per_step": wall / steps * 1e3, "event_ms_per_step": ev / steps * 1e3,
                "bytes_per_step": nbytes}

    def measure_shape(wtype, M, name, pool, reps=5):
        """one GEMV shape alone over every layer's distinct copy of it: HIP-event average per launch"""
        n, k = shapes[name]
        x = torch.randn((M, k), device="cuda", generator=gen).to(torch.bfloat16)
        y = torch.empty((M, n), dtype=torch.float32, device="cuda")
        ws = [layer[name] for layer in pool]
        if name == "gate_proj":
            ws += [layer["up_proj"] for layer in pool]

        def fn():
            for w in ws:
                ql.linear_q_gemv(w, x, None, ql.SCALE_X86_REF, out=y)
        replay = graphed(fn)
        _, ev = timed(replay, reps, 2)
        per = ev / (reps * len(ws))
        nbytes = synth.gemv_algorithmic_bytes(wtype, M, n, k, 2)
        return {"us": per * 1e6, "GBps": nbytes / per / 1e9, "bytes": nbytes, "launches": reps * len(ws)}

    wtype = ql.Q4_0 if args.wtype == "q4_0" else ql.Q8_0
    pool = make_pool(wtype, N_LAYERS)
    torch.cuda.synchronize()

    head = measure_workload(wtype, args.m, pool, args.steps, args.warmup)
    per_shape = {name: measure_shape(wtype, args.m, name, pool) for name in ("gate_proj", "down_proj", "q_proj", "o_proj", "k_proj")}
    dom = per_shape["gate_proj"]

    extra = {"per_shape": per_shape, "event_ms_per_step": head["event_ms_per_step"],
             "graph": not args.no_graph, "layers": N_LAYERS, "launches_per_step": N_LAYERS * len(shapes)}
    if not args.no_extra:
        for M in (4, 8):
            if M != args.m:
                r = measure_workload(wtype, M, pool, max(5, args.steps // 3), 2)
                extra["%s_m%d" % (args.wtype, M)] = {"GBps": r["GBps"], "ms_per_step": r["ms_per_step"],
                                                     "gate_proj": measure_shape(wtype, M, "gate_proj", pool, 3)}
        del pool
        torch.cuda.empty_cache()
        other = ql.Q8_0 if wtype == ql.Q4_0 else ql.Q4_0
        oname = "q8_0" if wtype == ql.Q4_0 else "q4_0"
        pool2 = make_pool(other, N_LAYERS)
        for M in (1, 4, 8):
            r = measure_workload(other, M, pool2, max(5, args.steps // 3), 2)
            extra["%s_m%d" % (oname, M)] = {"GBps": r["GBps"], "ms_per_step": r["ms_per_step"],
                                            "gate_proj": measure_shape(other, M, "gate_proj", pool2, 3)}
        del pool2
        torch.cuda.empty_cache()

    cpu = None
    if not args.no_cpu:
        from oracle import oracle as orc
        rng = synth.rng_for(1)
        otype = orc.Q4_0 if wtype == ql.Q4_0 else orc.Q8_0
        Ws = {name: synth.make_weight(rng, otype, n, k) for name, (n, k) in shapes.items()}
        xsf = {k: synth.make_x_bf16(rng, args.m, k)[1] for k in (2560, 4096, 9728)}
        cores = len(os.sched_getaffinity(0))
        threads = int(os.environ.get("OMP_NUM_THREADS", cores))
        for name, W in Ws.items():  # warm-up pass
            orc.linear_q(xsf[W.shape[1] * 32], W, otype)
        passes, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 10.0 and passes < 200:
            for name, W in Ws.items():
                orc.linear_q(xsf[W.shape[1] * 32], W, otype)
            passes += 1
        dt = time.perf_counter() - t0
        layer_bytes = step_bytes(wtype, args.m) / N_LAYERS
        cpu = {"value": layer_bytes * passes / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": "%d passes over ONE decoder layer (7 GEMVs, %.1f MB) with the C oracle "
                         "(scalar restatement of quantize_row_q8_0 + tinyBLAS block dots, OpenMP over output rows)"
                         % (passes, layer_bytes / 1e6)}

    out = {
        "metric": "W4 decode GEMV HBM GB/s" if wtype == ql.Q4_0 else "W8 decode GEMV HBM GB/s",
        "value": round(head["GBps"], 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Qwen3-4B decoder-layer decode GEMVs (q/k/v/o/gate/up/down), %s weights, bf16 x, M=%d; "
                               "one step = 36 layers x 7 projections = 252 launches over %.2f GB of distinct weights"
                               % (args.wtype.upper(), args.m, head["bytes_per_step"] / 1e9),
                   "M": args.m, "weights": args.wtype, "percent_of_hbm_peak": round(100 * head["GBps"] / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(dom["GBps"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom["GBps"] / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "gemv_q_kernel gate/up_proj N=9728 K=2560 M=%d" % args.m, "us_per_launch": round(dom["us"], 3),
                     "algorithmic_bytes_per_launch": dom["bytes"]},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
