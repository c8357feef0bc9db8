#!/usr/bin/env python3
"""Benchmark of the quantized-Linear hot path on one MI355X.

Workload (the configuration the metric is quoted on): the seven Linear projections of a Qwen3-4B decoder layer as decode
GEMVs with Q4_0 weights, bf16 activations, M = 1.  One step = one decode token through all 36 layers over 2.04 GB of
distinct weights (far larger than the 256 MB last-level cache, so every step streams from HBM).  Projections that read
the same activations share a launch (q/k/v, gate/up): 4 launches per layer, 144 per step; --per-op gives one launch per
projection (252 per step).  The launches of a step are captured once into a HIP graph and replayed.

Prints ONE JSON line.  `value` is whole-job algorithmic GB/s (weights 18 B per 32-element block + activations + outputs,
divided by wall time of the timed steps, inputs resident in HBM).  `roofline` is the dominant GEMV launch alone
(gate+up projection), timed with HIP events on the launch stream.  `cpu_baseline` times the CPU oracle of the same path on a
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
# counter summary of the dominant launch (two rocprofv3 --pmc runs of `bench.py --pmc-probe`); its "total" line is what
# roofline.traffic reports, so the figure and its evidence cannot drift apart
TRAFFIC_PROFILE = "profiles/gemv_q4_0_gate_up_m1_pmc_hbm_traffic.txt"


def traffic_from_profile():
    """bytes per launch from the committed counter summary (line `total  <bytes> B  vs algorithmic ...`), or None"""
    import re
    try:
        for line in open(os.path.join(ROOT, TRAFFIC_PROFILE)):
            m = re.match(r"\s*total\s+([0-9 ]+) B\s+vs algorithmic", line)
            if m:
                return int(m.group(1).replace(" ", ""))
    except OSError:
        pass
    return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--wtype", choices=["q4_0", "q8_0"], default="q4_0")
    ap.add_argument("--m", type=int, default=1, help="activation rows of the headline workload (1..8)")
    ap.add_argument("--per-op", action="store_true",
                    help="one launch per projection (7 per layer) instead of sibling projections sharing a launch (4 per layer)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="counter run: 20 launches of the dominant GEMV launch and 20 of a plain copy of the same byte count, "
                         "nothing else; meant to run under rocprofv3 --pmc FETCH_SIZE (or WRITE_SIZE)")
    ap.add_argument("--side-only", action="store_true",
                    help="profiling run: only the prefill GEMM / MoE side workloads (W8A8, W4A16, MoE FFN, Q4_0 prefill Linear), "
                         "printed as one JSON object; meant to run under rocprofv3")
    ap.add_argument("--brief", action="store_true",
                    help="with --side-only: one untimed and one timed replay per workload (counter runs: fewer dispatches to record)")
    ap.add_argument("--layer-only", action="store_true",
                    help="profiling run: only the decoder-layer chain (operators one by one and folded, M = 1 and 8), the "
                         "Q4_K / Q6_K gate projection at one row and the four launches of a Q4_K / Q6_K layer at eight, printed as one JSON object; meant to run under rocprofv3")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--request-order", type=int, default=-1, choices=[-1, 0, 1],
                    help="mllm_hip_gemv_set_request_order: -1 the library's rule (default), 0 / 1 never / always deferred (comparison runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the M=4/8 and Q8_0 side measurements")
    return ap.parse_args()


def side_workloads(torch, ql, synth, gen, brief=False):
    """The other configurations of the metric: W8A8 / W4A16 prefill GEMMs (MFMA-bound) and the MoE expert FFN."""
    WARM, TIMED = (1, 1) if brief else (3, 10)

    def ev_time(fn, reps):
        """seconds per call: `reps` calls captured in one HIP graph (a few microseconds of Python per eager call would otherwise
        be counted as kernel time of the small launches), replayed ten times between HIP events after three untimed replays
        (the first replays of a graph run 5 to 10 % slower than the steady state the headline's warm-up steps reach)"""
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(reps):
                fn()
        for _ in range(WARM):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(TIMED):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / (TIMED * reps)

    def ev_replay(g, reps):
        if brief:
            reps = 1
        for _ in range(WARM):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    out = {}
    # W8A8 prefill: A bf16 [2048,2048] with 1 % outliers x20, W int8 [6144,2048]
    M, N, K = 2048, 6144, 2048
    a = torch.randn((M, K), device="cuda", generator=gen)
    a = torch.where(torch.rand((M, K), device="cuda", generator=gen) < 0.01, a * 20, a).to(torch.bfloat16)
    Ws = [torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=gen) for _ in range(4)]
    ws = (torch.rand(N, device="cuda", generator=gen) + 0.01) * 0.01
    q, sc = ql.per_token_quant_int8(a)
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    wsp = torch.empty(_lib_ws(ql, "w8a8", M, K), dtype=torch.uint8, device="cuda")
    i = [0]

    def gemm():
        ql.w8a8_gemm(q, sc, Ws[i[0] % 4], ws, None, out=y)
        i[0] += 1

    def fused():
        ql.w8a8_linear(a, Ws[i[0] % 4], ws, None, workspace=wsp, out=y)
        i[0] += 1
    Wps = [ql.w8a8_prepack(w) for w in Ws]  # the load-time repack; the timed region reads packed weights only

    def gemm_p():
        ql.w8a8_gemm_packed(q, sc, Wps[i[0] % 4], N, ws, None, out=y)
        i[0] += 1

    def fused_p():
        ql.w8a8_linear_packed(a, Wps[i[0] % 4], N, ws, None, workspace=wsp, out=y)
        i[0] += 1
    tq = ev_time(lambda: ql.per_token_quant_int8(a), 20)
    tg, tf, tgp, tfp = ev_time(gemm, 20), ev_time(fused, 20), ev_time(gemm_p, 20), ev_time(fused_p, 20)
    ops = 2.0 * M * N * K
    out["w8a8_prefill_2048x6144x2048"] = {
        "gemm_us": tgp * 1e6, "gemm_TOPS": ops / tgp / 1e12, "gemm_frac_of_5000_TOPS": ops / tgp / 5e15,
        "quant_us": tq * 1e6, "quant_GBps": (M * K * 3 + M * 4) / tq / 1e9,
        "quant_plus_gemm_us": tfp * 1e6, "quant_plus_gemm_TOPS": ops / tfp / 1e12,
        "weights": "prepacked (mllm_hip_w8a8_prepack)",
        "plain_layout": {"gemm_us": tg * 1e6, "gemm_TOPS": ops / tg / 1e12, "quant_plus_gemm_us": tf * 1e6}}
    del Ws, Wps
    # W4A16 prefill: A bf16 [2048,2560], W uint4 [9728,2560] g128
    M, N, K = 2048, 9728, 2560
    a = torch.randn((M, K), device="cuda", generator=gen).to(torch.bfloat16)
    qws = [torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, device="cuda", generator=gen) for _ in range(3)]
    s4 = (torch.randn((N, K // 128), device="cuda", generator=gen).abs() * 0.01).to(torch.float16)
    zp = torch.randint(0, 256, (N, K // 256), dtype=torch.uint8, device="cuda", generator=gen)
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

    def g4():
        ql.w4a16_gemm(a, qws[i[0] % 3], s4, zp, None, 128, out=y)
        i[0] += 1
    pks = [ql.w4a16_prepack(qw, s4, zp, 128) for qw in qws]  # the load-time repack

    def g4p():
        ql.w4a16_gemm_packed(a, pks[i[0] % 3], N, None, 128, out=y)
        i[0] += 1
    t4, t4p = ev_time(g4, 10), ev_time(g4p, 10)
    fl = 2.0 * M * N * K
    out["w4a16_prefill_2048x9728x2560"] = {"us": t4p * 1e6, "TFLOPS": fl / t4p / 1e12, "frac_of_2500_TFLOPS": fl / t4p / 2.5e15,
                                           "weights": "prepacked (mllm_hip_w4a16_prepack)",
                                           "plain_layout": {"us": t4 * 1e6, "TFLOPS": fl / t4 / 1e12}}
    del qws, pks
    # MoE FFN: 512 tokens, hidden 2048, 128 experts, top-8 Zipf(1.1), intermediate 768, Q4_0
    import numpy as np
    T, H, I, E, k = 512, 2048, 768, 128, 8
    ids_np, w_np = synth.make_moe_routing(synth.rng_for(4), T, E, k)
    ids, tw = torch.from_numpy(ids_np).cuda(), torch.from_numpy(w_np).cuda()
    gate = ql.PackedExperts.synthetic(ql.Q4_0, E, I, H, gen)
    up = ql.PackedExperts.synthetic(ql.Q4_0, E, I, H, gen)
    down = ql.PackedExperts.synthetic(ql.Q4_0, E, H, I, gen)
    x = torch.randn((T, H), device="cuda", generator=gen).to(torch.bfloat16)
    wsm = torch.empty(_lib_ws(ql, "moe", T, H, I, E, k), dtype=torch.uint8, device="cuda")
    ym = torch.empty((T, H), dtype=torch.float32, device="cuda")
    tm = ev_time(lambda: ql.moe_ffn_q(gate, up, down, x, ids, tw, workspace=wsm, out=ym), 10)
    # the same layer with few tokens (1 and 8: decode; 16 and 32: short batches, still at most three pairs per expert): every
    # (token, expert) pair a GEMV row, two launches; a graph of 16 calls over rotating routings (eager launches of this size
    # would measure the host)
    dec = {}
    for Td in (1, 8, 16, 32):
        rngd = synth.rng_for(4, 100 + Td)
        routes = [synth.make_moe_routing(rngd, Td, E, k) for _ in range(16)]
        idl = [torch.from_numpy(r[0]).cuda() for r in routes]
        twl = [torch.from_numpy(r[1]).cuda() for r in routes]
        xd = torch.randn((Td, H), device="cuda", generator=gen).to(torch.bfloat16)
        yd = torch.empty((Td, H), dtype=torch.float32, device="cuda")

        def dstep():
            for i_, t_ in zip(idl, twl):
                ql.moe_ffn_q(gate, up, down, xd, i_, t_, workspace=wsm, out=yd)
        dstep()
        torch.cuda.synchronize()
        gd = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gd):
            dstep()
        td = ev_replay(gd, 10) / 16
        act = float(np.mean([len(np.unique(r[0])) for r in routes]))
        wb = act * (2 * I * (H // 32) * 18 + H * (I // 32) * 18)
        dec["tokens_%d" % Td] = {"us": td * 1e6, "active_experts_avg": act, "weight_GBps": wb / td / 1e9, "frac_of_hbm_peak": wb / td / 8e12}
    del gate, up, down
    # the router gate of that layer (MoEGate::forward: logits, softmax, the k largest, weights): fp32 gate weights [E, H], 16
    # distinct copies, with a scores buffer (two launches) and without (one workgroup per four tokens)
    gws = [torch.randn((E, H), device="cuda", generator=gen) * 0.05 for _ in range(16)]
    gatet = {}
    for Tg in (1, 8, 512):
        xg = torch.randn((Tg, H), device="cuda", generator=gen).to(torch.bfloat16)
        scb = torch.empty((Tg, E), dtype=torch.float32, device="cuda")
        t2 = ev_time(lambda: [ql.moe_gate(xg, w_, k, scores=scb) for w_ in gws], 1) / 16
        t1 = ev_time(lambda: [ql.moe_gate(xg, w_, k) for w_ in gws], 1) / 16
        gatet["tokens_%d" % Tg] = {"us": t2 * 1e6, "one_launch_us": t1 * 1e6}
    del gws
    # the same layer with Q4_K experts (the format of the shipped Qwen3-MoE recipe), 1 and 8 tokens: pairs as K-quant GEMV rows
    gk = ql.PackedKExperts.synthetic(ql.Q4_K, E, I, H, gen)
    uk = ql.PackedKExperts.synthetic(ql.Q4_K, E, I, H, gen)
    dk = ql.PackedKExperts.synthetic(ql.Q4_K, E, H, I, gen)
    deck = {}
    for Td in (1, 8):
        rngd = synth.rng_for(4, 100 + Td)
        routes = [synth.make_moe_routing(rngd, Td, E, k) for _ in range(16)]
        idl = [torch.from_numpy(r[0]).cuda() for r in routes]
        twl = [torch.from_numpy(r[1]).cuda() for r in routes]
        xd = torch.randn((Td, H), device="cuda", generator=gen).to(torch.bfloat16)
        yd = torch.empty((Td, H), dtype=torch.float32, device="cuda")
        from mllm_amd import _lib as _l
        wsk = torch.empty(_l.lib().mllm_hip_moe_kq_workspace_bytes(Td, H, I, E, k), dtype=torch.uint8, device="cuda")

        def kstep():
            for i_, t_ in zip(idl, twl):
                ql.moe_ffn_kq(gk, uk, dk, xd, i_, t_, workspace=wsk, out=yd)
        kstep()
        torch.cuda.synchronize()
        gd = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gd):
            kstep()
        td = ev_replay(gd, 10) / 16
        act = float(np.mean([len(np.unique(r[0])) for r in routes]))
        wb = act * 3 * I * (H // 256) * 144
        deck["tokens_%d" % Td] = {"us": td * 1e6, "active_experts_avg": act, "weight_GBps": wb / td / 1e9, "frac_of_hbm_peak": wb / td / 8e12}
    # the 512-token layer with Q4_K experts: pairs sorted by expert, tiles of 32 rows on the matrix cores (the grouped form),
    # against tiles of eight rows (the decode kernels) and one GEMV row per pair
    from mllm_amd import _lib as _l
    wsk = torch.empty(_l.lib().mllm_hip_moe_kq_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device="cuda")
    tk2 = ev_time(lambda: ql.moe_ffn_kq(gk, uk, dk, x, ids, tw, workspace=wsk, out=ym), 5)
    _l.lib().mllm_hip_moe_kq_set_path(2)
    tk8 = ev_time(lambda: ql.moe_ffn_kq(gk, uk, dk, x, ids, tw, workspace=wsk, out=ym), 5)
    _l.lib().mllm_hip_moe_kq_set_path(1)
    tk1 = ev_time(lambda: ql.moe_ffn_kq(gk, uk, dk, x, ids, tw, workspace=wsk, out=ym), 3)
    _l.lib().mllm_hip_moe_kq_set_path(0)
    wbk = int((np.bincount(ids_np.reshape(-1), minlength=E) > 0).sum()) * 3 * I * (H // 256) * 144
    # the shipped recipe's formats: gate / up Q4_K, down Q6_K (examples/qwen3_moe/quant_cfg_30B_q4_k.json)
    dk6 = ql.PackedKExperts.synthetic(ql.Q6_K, E, H, I, gen)
    tk6 = ev_time(lambda: ql.moe_ffn_kq(gk, uk, dk6, x, ids, tw, workspace=wsk, out=ym), 5)
    wbk6 = wbk // 3 * 2 + int((np.bincount(ids_np.reshape(-1), minlength=E) > 0).sum()) * H * (I // 256) * 210
    deck["tokens_512_grouped_q4_k_gate_up_q6_k_down"] = {"us": tk6 * 1e6, "weight_GBps": wbk6 / tk6 / 1e9,
                                                         "frac_of_hbm_peak": wbk6 / tk6 / 8e12}
    del dk6
    deck["tokens_512_grouped"] = {"us": tk2 * 1e6, "weight_GBps": wbk / tk2 / 1e9, "frac_of_hbm_peak": wbk / tk2 / 8e12,
                                  "tiles_of_8_rows_us": tk8 * 1e6, "pairs_as_gemv_rows_us": tk1 * 1e6}
    del gk, uk, dk, wsk
    from mllm_amd import _lib
    L = _lib.lib()
    gate2 = ql.PackedExperts.synthetic(ql.Q4_0, E, I, H, gen, layout="gemm")
    up2 = ql.PackedExperts.synthetic(ql.Q4_0, E, I, H, gen, layout="gemm")
    down2 = ql.PackedExperts.synthetic(ql.Q4_0, E, H, I, gen, layout="gemm")
    wsm2 = torch.empty(L.mllm_hip_moe_gemm_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device="cuda")
    tm2 = ev_time(lambda: ql.moe_ffn_q_gemm(gate2, up2, down2, x, ids, tw, workspace=wsm2, out=ym), 10)
    L.mllm_hip_moe_gemm_set_path(1)
    tm3 = ev_time(lambda: ql.moe_ffn_q_gemm(gate2, up2, down2, x, ids, tw, workspace=wsm2, out=ym), 10)
    L.mllm_hip_moe_gemm_set_path(0)
    active = int((np.bincount(ids_np.reshape(-1), minlength=E) > 0).sum())
    wbytes = active * (2 * I * (H // 32) * 18 + H * (I // 32) * 18)
    flops = T * k * (2.0 * H * I * 2 + 2.0 * I * H)
    out["moe_ffn_512tok_128e_top8_q4_0"] = {"us": tm2 * 1e6, "active_experts": active, "weight_GBps": wbytes / tm2 / 1e9,
                                            "frac_of_hbm_peak": wbytes / tm2 / 8e12, "TFLOPS": flops / tm2 / 1e12,
                                            "path": "mllm_hip_moe_ffn_q_gemm, default form: the reference's block arithmetic on the matrix "
                                                    "cores (exact integer block sums and exact scale products from fp16 MFMAs, one fp32 FMA "
                                                    "per block; 4 launches: route + quantize, gate + up + SiLU*up + re-quantize, down, weighted sum)",
                                            "fp16_operand_form": {"us": tm3 * 1e6, "weight_GBps": wbytes / tm3 / 1e9,
                                                                  "note": "mllm_hip_moe_gemm_set_path(1): block scales folded into fp16 "
                                                                          "operands, no exact block sums (about 2e-4 from the oracle)"},
                                            "block_dot_path": {"us": tm * 1e6, "weight_GBps": wbytes / tm / 1e9,
                                                               "note": "mllm_hip_moe_ffn_q: int8 MFMA block sums scaled on the vector ALU"},
                                            "decode": dec, "decode_q4_k_experts": deck, "router_gate": gatet}
    del gate2, up2, down2
    # Q4_0 Linear at prefill size (the reference's tinyBLAS gemm branch): gate_proj of the decode layer, 2048 rows
    M, N, K = 2048, 9728, 2560
    xx = torch.randn((M, K), device="cuda", generator=gen).to(torch.bfloat16)
    yy = torch.empty((M, N), dtype=torch.float32, device="cuda")
    wv = ql.PackedQWeight.synthetic(ql.Q4_0, N, K, gen)
    wg = ql.PackedQWeight.synthetic(ql.Q4_0, N, K, gen, layout="gemm")
    ws1 = torch.empty(L.mllm_hip_linear_q_workspace_bytes(M, K), dtype=torch.uint8, device="cuda")
    ws2 = torch.empty(L.mllm_hip_linear_q_gemm_workspace_bytes(M, K), dtype=torch.uint8, device="cuda")
    t1 = ev_time(lambda: ql.linear_q(wv, xx, None, ql.SCALE_X86_REF, workspace=ws1, out=yy), 5)
    t2 = ev_time(lambda: ql.linear_q_gemm(wg, xx, None, ql.SCALE_X86_REF, workspace=ws2, out=yy), 10)
    fl = 2.0 * M * N * K
    out["q4_0_linear_prefill_2048x9728x2560"] = {"us": t2 * 1e6, "TFLOPS": fl / t2 / 1e12, "frac_of_2500_TFLOPS": fl / t2 / 2.5e15,
                                                  "path": "matrix cores (mllm_hip_linear_q_gemm)",
                                                  "block_dot_path": {"us": t1 * 1e6, "TOPS": fl / t1 / 1e12}}
    del wv
    # a short prompt: 128 rows through the gate and the down projection of the layer; K cut into ranges (the _short entry point)
    # against one workgroup per tile
    sp = {}
    for nm, (n_, k_) in (("gate_9728x2560", (9728, 2560)), ("down_2560x9728", (2560, 9728))):
        wsg = wg if (n_, k_) == (N, K) else ql.PackedQWeight.synthetic(ql.Q4_0, n_, k_, gen, layout="gemm")
        xs_ = torch.randn((128, k_), device="cuda", generator=gen).to(torch.bfloat16)
        ys_ = torch.empty((128, n_), dtype=torch.float32, device="cuda")
        wss = torch.empty(L.mllm_hip_linear_q_gemm_short_workspace_bytes(128, n_, k_), dtype=torch.uint8, device="cuda")
        ta = ev_time(lambda: ql.linear_q_gemm(wsg, xs_, None, ql.SCALE_X86_REF, workspace=wss, out=ys_), 10)
        tb = ev_time(lambda: ql.linear_q_gemm(wsg, xs_, None, ql.SCALE_X86_REF, workspace=wss, out=ys_, short=True), 10)
        sp[nm] = {"us": tb * 1e6, "one_workgroup_per_tile_us": ta * 1e6}
    out["q4_0_linear_short_prompt_128_rows"] = sp
    del wg
    # the same Linear with Q4_K / Q6_K weights (Q8_K activations): matrix cores against passes of the eight-row GEMV
    for kname, kt in (("q4_k", ql.Q4_K), ("q6_k", ql.Q6_K)):
        wkg = ql.PackedKWeight.synthetic(kt, N, K, gen, layout="gemm")
        wsk = torch.empty(L.mllm_hip_linear_kq_gemm_workspace_bytes(M, K), dtype=torch.uint8, device="cuda")
        tk = ev_time(lambda: ql.linear_kq_gemm(wkg, xx, out=yy, workspace=wsk), 10)
        wkv = ql.PackedKWeight.synthetic(kt, N, K, gen)
        wsv = ql.kq_workspace(M, K, N)
        tv = ev_time(lambda: ql.linear_kq(wkv, xx, out=yy, workspace=wsv), 3)
        out["%s_linear_prefill_2048x9728x2560" % kname] = {"us": tk * 1e6, "TFLOPS": fl / tk / 1e12, "frac_of_2500_TFLOPS": fl / tk / 2.5e15,
                                                            "path": "matrix cores (mllm_hip_linear_kq_gemm)",
                                                            "gemv_passes_path": {"us": tv * 1e6}}
        del wkg, wkv
    # W8A8 / W4A16 at decode size (the GEMV kernels against packed weights; W8A8 with its per-token quantization) and the
    # operators of a decode token around the Linears
    dec_ops = {}
    for nm, (n_, k_) in (("gate_9728x2560", (9728, 2560)), ("down_2560x9728", (2560, 9728))):
        Wp8 = [ql.w8a8_prepack(torch.randint(-127, 128, (n_, k_), dtype=torch.int8, device="cuda", generator=gen)) for _ in range(4)]
        ws8 = (torch.rand(n_, device="cuda", generator=gen) + 0.01) * 0.01
        s4 = (torch.randn((n_, k_ // 128), device="cuda", generator=gen).abs() * 0.01).to(torch.float16)
        zp = torch.randint(0, 256, (n_, k_ // 256), dtype=torch.uint8, device="cuda", generator=gen)
        Wp4 = [ql.w4a16_prepack(torch.randint(0, 256, (n_, k_ // 2), dtype=torch.uint8, device="cuda", generator=gen), s4, zp, 128)
               for _ in range(4)]
        for m_ in (1, 4, 8, 16):
            a_ = torch.randn((m_, k_), device="cuda", generator=gen).to(torch.bfloat16)
            y_ = torch.empty((m_, n_), dtype=torch.bfloat16, device="cuda")
            wq = torch.empty(_lib_ws(ql, "w8a8", m_, k_), dtype=torch.uint8, device="cuda")
            j = [0]

            def f8():
                ql.w8a8_linear_packed(a_, Wp8[j[0] % 4], n_, ws8, None, workspace=wq, out=y_)
                j[0] += 1

            def f4():
                ql.w4a16_gemm_packed(a_, Wp4[j[0] % 4], n_, None, 128, out=y_)
                j[0] += 1
            t8, t4 = ev_time(f8, 8), ev_time(f4, 8)
            dec_ops["%s_tokens_%d" % (nm, m_)] = {"w8a8_us": t8 * 1e6, "w8a8_weight_GBps": n_ * k_ / t8 / 1e9,
                                                  "w4a16_us": t4 * 1e6, "w4a16_weight_GBps": n_ * k_ / 2 / t4 / 1e9}
        del Wp8, Wp4
    xs_ = torch.randn((8, 151936), device="cuda", generator=gen)
    dec_ops["softmax_8x151936_us"] = ev_time(lambda: ql.softmax(xs_), 2) * 1e6
    dec_ops["topk_20_of_151936_us"] = ev_time(lambda: ql.topk(xs_[:1], 20), 2) * 1e6
    xs_ = torch.randn((32 * 512, 512), device="cuda", generator=gen)
    dec_ops["softmax_16384x512_us"] = ev_time(lambda: ql.softmax(xs_), 8) * 1e6
    xs_ = torch.randn((512, 128), device="cuda", generator=gen)
    dec_ops["topk_8_of_128_rows_512_us"] = ev_time(lambda: ql.topk(xs_, 8), 8) * 1e6
    p_ = torch.randn((32, 1, 8192), device="cuda", generator=gen).to(torch.bfloat16)
    v_ = torch.randn((32, 8192, 128), device="cuda", generator=gen).to(torch.bfloat16)
    o_ = torch.empty((32, 1, 128), dtype=torch.bfloat16, device="cuda")
    tpv = ev_time(lambda: ql.matmul(p_, v_, out=o_), 8)
    dec_ops["matmul_scores_x_values_32x1x8192x128_bf16"] = {"us": tpv * 1e6, "GBps": v_.numel() * 2 / tpv / 1e9}
    s_ = torch.empty((32, 1, 8192), dtype=torch.bfloat16, device="cuda")
    q_ = torch.randn((32, 1, 128), device="cuda", generator=gen).to(torch.bfloat16)
    tqk = ev_time(lambda: ql.matmul(q_, v_, transpose_b=True, out=s_), 8)
    dec_ops["matmul_query_x_keys_32x1x128x8192_bf16"] = {"us": tqk * 1e6, "GBps": v_.numel() * 2 / tqk / 1e9}
    out["decode_size_w8a8_w4a16_and_operators"] = dec_ops
    return out


def _lib_ws(ql, which, *a):
    from mllm_amd import _lib
    L = _lib.lib()
    return L.mllm_hip_w8a8_workspace_bytes(*a) if which == "w8a8" else L.mllm_hip_moe_workspace_bytes(*a)


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
    _lib.check(_lib.lib().mllm_hip_gemv_set_request_order(args.request_order), "mllm_hip_gemv_set_request_order")
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(synth.SEED_BASE + 1)
    shapes = synth.QWEN3_4B_LAYER
    stream = torch.cuda.current_stream()
    if args.side_only:
        print(json.dumps({"side_only": True, "prefill_and_moe": side_workloads(torch, ql, synth, gen, brief=args.brief)}))
        return

    def make_pool(wtype, layers):
        return [{name: ql.PackedQWeight.synthetic(wtype, n, k, gen) for name, (n, k) in shapes.items()}
                for _ in range(layers)]

    def make_io(M):
        xs = {k: torch.randn((M, k), device="cuda", generator=gen).to(torch.bfloat16) for k in (2560, 4096, 9728)}
        # room for the K slices' partial sums of the widest launch that reads x of this length (gate + up: 2 x 9728 rows)
        n_total = {2560: 2 * 9728, 4096: 2560, 9728: 2560}
        xs["workspaces"] = {k: (ql.gemv_workspace(M, k, n_total[k]) if M >= 3 else None) for k in (2560, 4096, 9728)}
        ys = {name: torch.empty((M, n), dtype=torch.float32, device="cuda") for name, (n, _) in shapes.items()}
        return xs, ys

    def step_bytes(wtype, M):
        return N_LAYERS * sum(synth.gemv_algorithmic_bytes(wtype, M, n, k, 2) for n, k in shapes.values())

    def run_step(pool, xs, ys):
        """one decode token: per layer q/k/v in one launch, o, gate/up in one launch, down (4 launches)"""
        if args.per_op:
            for layer in pool:
                for name, w in layer.items():
                    ql.linear_q_gemv(w, xs[w.K], None, ql.SCALE_X86_REF, out=ys[name])
            return
        # from three activation rows on the calls get a workspace with room for the partial sums of the K slices
        wk = xs["workspaces"]
        for l in pool:
            ql.linear_q_gemv_multi([l["q_proj"], l["k_proj"], l["v_proj"]], xs[2560], None, ql.SCALE_X86_REF,
                                   [ys["q_proj"], ys["k_proj"], ys["v_proj"]], workspace=wk[2560])
            ql.linear_q_gemv_multi([l["o_proj"]], xs[4096], None, ql.SCALE_X86_REF, [ys["o_proj"]], workspace=wk[4096])
            ql.linear_q_gemv_multi([l["gate_proj"], l["up_proj"]], xs[2560], None, ql.SCALE_X86_REF,
                                   [ys["gate_proj"], ys["up_proj"]], workspace=wk[2560])
            ql.linear_q_gemv_multi([l["down_proj"]], xs[9728], None, ql.SCALE_X86_REF, [ys["down_proj"]], workspace=wk[9728])

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
        """one GEMV launch shape alone over every layer's distinct copy of it: HIP-event average per launch.
        "gate_up" / "qkv" are the sibling launches (two / three matrices, one launch)."""
        groups = {"gate_up": ["gate_proj", "up_proj"], "qkv": ["q_proj", "k_proj", "v_proj"]}.get(name, [name])
        k = shapes[groups[0]][1]
        x = torch.randn((M, k), device="cuda", generator=gen).to(torch.bfloat16)
        ys = [torch.empty((M, shapes[g][0]), dtype=torch.float32, device="cuda") for g in groups]
        sets = [[layer[g] for g in groups] for layer in pool]
        if name == "gate_proj":
            sets += [[layer["up_proj"]] for layer in pool]

        # three rows or more: with the workspace the step uses (room for the partial sums of the K slices)
        wsp = ql.gemv_workspace(M, k, sum(shapes[g][0] for g in groups)) if M >= 3 else None

        def fn():
            for ws in sets:
                if len(ws) == 1 and wsp is None:
                    ql.linear_q_gemv(ws[0], x, None, ql.SCALE_X86_REF, out=ys[0])
                else:
                    ql.linear_q_gemv_multi(ws, x, None, ql.SCALE_X86_REF, ys, workspace=wsp)
        replay = graphed(fn)
        _, ev = timed(replay, reps, 2)
        per = ev / (reps * len(sets))
        nbytes = sum(synth.gemv_algorithmic_bytes(wtype, M, shapes[g][0], k, 2) for g in groups) - (len(groups) - 1) * M * k * 2
        return {"us": per * 1e6, "GBps": nbytes / per / 1e9, "bytes": nbytes, "launches": reps * len(sets)}

    def measure_layer_chain(pool, M, reps=5):
        """The dependent chain of one decoder layer around its Linears (attention core left out: o_proj reads a fixed
        buffer), fp32 residual stream, over all layers: the operators one by one (10 launches per layer) against the
        folded form (RMSNorm and SiLU*up write the GEMV's quantized image, residual adds in the GEMV epilogue: 7), and with
        gate / up / SiLU / product / image as one launch (6)."""
        x0 = torch.randn((M, 2560), device="cuda", generator=gen)
        attn = torch.randn((M, 4096), device="cuda", generator=gen)
        nw = [torch.ones(2560, device="cuda") for _ in range(2)]
        b = {n: torch.empty((M, d), dtype=torch.float32, device="cuda")
             for n, d in (("h", 2560), ("q", 4096), ("k", 1024), ("v", 1024), ("o", 2560), ("x1", 2560), ("h2", 2560),
                          ("g", 9728), ("u", 9728), ("s", 9728), ("a", 9728), ("d", 2560), ("x2", 2560))}
        img = {k: ql.gemv_workspace(M, k) for k in (2560, 9728)}
        ws_o = ql.gemv_workspace(M, 4096, 2560)  # o_proj reads the attention output raw
        # room for the partial sums of the K slices (three rows or more: the slices of a row tile are separate workgroups)
        wsp = {2560: ql.gemv_workspace(M, 2560, 2 * 9728), 9728: ql.gemv_workspace(M, 9728, 2560)} if M >= 3 else {2560: None, 9728: None}
        L = _lib.lib()

        def ew(fn, a_, b_, y_):
            _lib.check(fn(a_.data_ptr(), b_.data_ptr(), y_.data_ptr(), 0, a_.shape[0], a_.shape[1], None, 0,
                          torch.cuda.current_stream().cuda_stream), "ew")

        def plain():
            x = x0
            for l in pool:
                ql.rmsnorm(x, nw[0], 1e-6, out=b["h"])
                ql.linear_q_gemv_multi([l["q_proj"], l["k_proj"], l["v_proj"]], b["h"], None, ql.SCALE_X86_REF, [b["q"], b["k"], b["v"]])
                ql.linear_q_gemv(l["o_proj"], attn, None, ql.SCALE_X86_REF, out=b["o"])
                ew(L.mllm_hip_add, b["o"], x, b["x1"])
                ql.rmsnorm(b["x1"], nw[1], 1e-6, out=b["h2"])
                ql.linear_q_gemv_multi([l["gate_proj"], l["up_proj"]], b["h2"], None, ql.SCALE_X86_REF, [b["g"], b["u"]])
                _lib.check(L.mllm_hip_silu(b["g"].data_ptr(), b["s"].data_ptr(), 0, b["g"].numel(),
                                           torch.cuda.current_stream().cuda_stream), "silu")
                ew(L.mllm_hip_mul, b["s"], b["u"], b["a"])
                ql.linear_q_gemv(l["down_proj"], b["a"], None, ql.SCALE_X86_REF, out=b["d"])
                ew(L.mllm_hip_add, b["d"], b["x1"], b["x2"])
                x = b["x2"]

        def folded():
            x = x0
            for l in pool:
                st = torch.cuda.current_stream().cuda_stream
                _lib.check(L.mllm_hip_rmsnorm(x.data_ptr(), 0, nw[0].data_ptr(), b["h"].data_ptr(), M, 2560, 1e-6, 0,
                                              img[2560].data_ptr(), ql.SCALE_X86_REF, st), "rmsnorm")
                ql.linear_q_gemv_fused([l["q_proj"], l["k_proj"], l["v_proj"]], img[2560], M=M, image=True, outs=[b["q"], b["k"], b["v"]],
                                       workspace=wsp[2560])
                ql.linear_q_gemv_fused([l["o_proj"]], attn, residuals=[x], outs=[b["x1"]], workspace=ws_o)
                _lib.check(L.mllm_hip_rmsnorm(b["x1"].data_ptr(), 0, nw[1].data_ptr(), b["h2"].data_ptr(), M, 2560, 1e-6, 0,
                                              img[2560].data_ptr(), ql.SCALE_X86_REF, st), "rmsnorm")
                ql.linear_q_gemv_fused([l["gate_proj"], l["up_proj"]], img[2560], M=M, image=True, outs=[b["g"], b["u"]], workspace=wsp[2560])
                _lib.check(L.mllm_hip_silu_mul(b["g"].data_ptr(), b["u"].data_ptr(), b["a"].data_ptr(), 0, M, 9728,
                                               img[9728].data_ptr(), ql.SCALE_X86_REF, st), "silu_mul")
                ql.linear_q_gemv_fused([l["down_proj"]], img[9728], M=M, image=True, residuals=[b["x1"]], outs=[b["x2"]], workspace=wsp[9728])
                x = b["x2"]

        def mlp_one_launch():
            x = x0
            for l in pool:
                st = torch.cuda.current_stream().cuda_stream
                _lib.check(L.mllm_hip_rmsnorm(x.data_ptr(), 0, nw[0].data_ptr(), b["h"].data_ptr(), M, 2560, 1e-6, 0,
                                              img[2560].data_ptr(), ql.SCALE_X86_REF, st), "rmsnorm")
                ql.linear_q_gemv_fused([l["q_proj"], l["k_proj"], l["v_proj"]], img[2560], M=M, image=True, outs=[b["q"], b["k"], b["v"]],
                                       workspace=wsp[2560])
                ql.linear_q_gemv_fused([l["o_proj"]], attn, residuals=[x], outs=[b["x1"]], workspace=ws_o)
                _lib.check(L.mllm_hip_rmsnorm(b["x1"].data_ptr(), 0, nw[1].data_ptr(), b["h2"].data_ptr(), M, 2560, 1e-6, 0,
                                              img[2560].data_ptr(), ql.SCALE_X86_REF, st), "rmsnorm")
                _lib.check(L.mllm_hip_mlp_gate_up_q(l["gate_proj"].wtype, l["gate_proj"].ptr, l["up_proj"].ptr, img[2560].data_ptr(),
                                                    ql.Q8_IMAGE, None, img[9728].data_ptr(), M, 9728, 2560, ql.SCALE_X86_REF, st), "mlp")
                ql.linear_q_gemv_fused([l["down_proj"]], img[9728], M=M, image=True, residuals=[b["x1"]], outs=[b["x2"]], workspace=wsp[9728])
                x = b["x2"]
        res = {}
        for name, fn, n in (("operators_one_by_one", plain, 10), ("folded", folded, 7), ("folded_mlp_one_launch", mlp_one_launch, 6)):
            _, ev = timed(graphed(fn), reps, 2)
            res[name] = {"us_per_layer": ev / (reps * len(pool)) * 1e6, "launches_per_layer": n}
        return res

    wtype = ql.Q4_0 if args.wtype == "q4_0" else ql.Q8_0
    if args.pmc_probe:
        pool = make_pool(wtype, 20)
        x = torch.randn((args.m, 2560), device="cuda", generator=gen).to(torch.bfloat16)
        ys = [torch.empty((args.m, 9728), dtype=torch.float32, device="cuda") for _ in range(2)]
        nbytes = 2 * synth.gemv_algorithmic_bytes(wtype, args.m, 9728, 2560, 2) // 16 * 16
        src = torch.randint(0, 255, (20, nbytes), dtype=torch.uint8, device="cuda", generator=gen)
        dst = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        for l in pool:
            ql.linear_q_gemv_multi([l["gate_proj"], l["up_proj"]], x, None, ql.SCALE_X86_REF, ys)
        for i in range(20):
            _lib.check(_lib.lib().mllm_hip_probe_copy(dst.data_ptr(), src[i].data_ptr(), nbytes, stream.cuda_stream), "probe_copy")
        torch.cuda.synchronize()
        print(json.dumps({"pmc_probe": True, "gemv_algorithmic_bytes": nbytes, "copy_bytes_read": nbytes, "copy_bytes_written": nbytes}))
        return
    pool = make_pool(wtype, N_LAYERS)
    torch.cuda.synchronize()
    if args.layer_only:
        res = {"layer_only": True, "decode_layer_chain": {"m%d" % M: measure_layer_chain(pool, M, reps=3) for M in (1, 8)}}
        x1 = torch.randn((1, 2560), device="cuda", generator=gen).to(torch.bfloat16)
        y1 = torch.empty((1, 9728), dtype=torch.float32, device="cuda")
        for kname, kt in (("q4_k", ql.Q4_K), ("q6_k", ql.Q6_K)):
            ws = [ql.PackedKWeight.synthetic(kt, 9728, 2560, gen) for _ in range(N_LAYERS)]
            _, ev = timed(graphed(lambda: [ql.linear_kq(w, x1, out=y1) for w in ws]), 3, 2)
            res["%s_gate_proj_us" % kname] = ev / (3 * N_LAYERS) * 1e6
            del ws
            # the four launches of a layer (q+k+v | o | gate+up | down) at eight rows over 12 layers' weights, with workspaces
            # that have room for the partial sums of K slices
            kpool = [{name: ql.PackedKWeight.synthetic(kt, n, k, gen) for name, (n, k) in shapes.items()} for _ in range(12)]
            xs8 = {k: torch.randn((8, k), device="cuda", generator=gen).to(torch.bfloat16) for k in (2560, 4096, 9728)}
            ys8 = {name: torch.empty((8, n), dtype=torch.float32, device="cuda") for name, (n, _) in shapes.items()}
            kws = {k: ql.kq_workspace(8, k, 2 * 9728) for k in (2560, 4096, 9728)}

            def klayers():
                for l in kpool:
                    ql.linear_kq_multi([l["q_proj"], l["k_proj"], l["v_proj"]], xs8[2560], None, [ys8["q_proj"], ys8["k_proj"], ys8["v_proj"]],
                                       workspace=kws[2560])
                    ql.linear_kq(l["o_proj"], xs8[4096], out=ys8["o_proj"], workspace=kws[4096])
                    ql.linear_kq_multi([l["gate_proj"], l["up_proj"]], xs8[2560], None, [ys8["gate_proj"], ys8["up_proj"]], workspace=kws[2560])
                    ql.linear_kq(l["down_proj"], xs8[9728], out=ys8["down_proj"], workspace=kws[9728])
            _, ev = timed(graphed(klayers), 3, 2)
            res["%s_layer_m8_us" % kname] = ev / (3 * 12) * 1e6
            del kpool
        print(json.dumps(res))
        return

    head = measure_workload(wtype, args.m, pool, args.steps, args.warmup)
    per_shape = {name: measure_shape(wtype, args.m, name, pool)
                 for name in ("gate_up", "qkv", "gate_proj", "down_proj", "q_proj", "o_proj", "k_proj")}
    dom_name = "gate_proj" if args.per_op else "gate_up"
    dom = per_shape[dom_name]
    # BASELINE configs[0]: the single Q4_0 Linear [1,2048] x [6144,2048]^T with fp32 activations, over 80 distinct copies of the
    # weight (566 MB: every launch streams from HBM), one launch each
    c1w = [ql.PackedQWeight.synthetic(ql.Q4_0, 6144, 2048, gen) for _ in range(80)]
    c1x = torch.randn((1, 2048), device="cuda", generator=gen)
    c1y = torch.empty((1, 6144), dtype=torch.float32, device="cuda")
    _, ev = timed(graphed(lambda: [ql.linear_q_gemv(w, c1x, None, ql.SCALE_X86_REF, out=c1y) for w in c1w]), 5, 2)
    c1b = synth.gemv_algorithmic_bytes(ql.Q4_0, 1, 6144, 2048, 4)
    per_shape["c1_6144x2048_fp32_x"] = {"us": ev / (5 * 80) * 1e6, "GBps": c1b / (ev / (5 * 80)) / 1e9, "bytes": c1b, "launches": 400}
    del c1w

    extra = {"per_shape": per_shape, "event_ms_per_step": head["event_ms_per_step"],
             "graph": not args.no_graph, "layers": N_LAYERS, "launches_per_step": N_LAYERS * (len(shapes) if args.per_op else 4)}
    if not args.no_extra:
        extra["decode_layer_chain"] = {"m%d" % M: measure_layer_chain(pool, M) for M in (1, 4, 8)}
        for M in (2, 4, 8):
            if M != args.m:
                r = measure_workload(wtype, M, pool, max(5, args.steps // 3), 2)
                extra["%s_m%d" % (args.wtype, M)] = {"GBps": r["GBps"], "ms_per_step": r["ms_per_step"],
                                                     dom_name: measure_shape(wtype, M, dom_name, pool, 3)}
        # short batches: the whole groups of eight rows share a launch (weights read from memory once per launch)
        for M in (16, 32):
            if M != args.m:
                r = measure_workload(wtype, M, pool, max(5, args.steps // 3), 2)
                extra["%s_m%d" % (args.wtype, M)] = {"GBps": r["GBps"], "ms_per_step": r["ms_per_step"],
                                                     "rows_per_ms": M / r["ms_per_step"]}
        del pool
        torch.cuda.empty_cache()
        other = ql.Q8_0 if wtype == ql.Q4_0 else ql.Q4_0
        oname = "q8_0" if wtype == ql.Q4_0 else "q4_0"
        pool2 = make_pool(other, N_LAYERS)
        for M in (1, 2, 4, 8):
            r = measure_workload(other, M, pool2, max(5, args.steps // 3), 2)
            extra["%s_m%d" % (oname, M)] = {"GBps": r["GBps"], "ms_per_step": r["ms_per_step"],
                                            dom_name: measure_shape(other, M, dom_name, pool2, 3)}
        del pool2
        torch.cuda.empty_cache()

    if not args.no_extra:
        # Q4_K / Q6_K weights (the formats of the shipped Qwen3-MoE recipe) on the same layer shapes and launch plan as the
        # headline workload (144 launches per step), Q8_K activation quantization inside the kernel
        kq = {}
        for kname, kt, bb in (("q4_k", ql.Q4_K, 144), ("q6_k", ql.Q6_K, 210)):
            kpool = [{name: ql.PackedKWeight.synthetic(kt, n, k, gen) for name, (n, k) in shapes.items()} for _ in range(N_LAYERS)]
            for M in (1, 8):
                xs, ys = make_io(M)
                kws = {k: ql.kq_workspace(M, k, 2 * 9728) for k in (2560, 4096, 9728)}  # (with room for partial sums of K slices)

                def kstep():  # sibling projections share a launch: qkv | o | gate+up | down
                    for l in kpool:
                        ql.linear_kq_multi([l["q_proj"], l["k_proj"], l["v_proj"]], xs[2560], None, [ys["q_proj"], ys["k_proj"], ys["v_proj"]],
                                           workspace=kws[2560])
                        ql.linear_kq(l["o_proj"], xs[4096], out=ys["o_proj"], workspace=kws[4096])
                        ql.linear_kq_multi([l["gate_proj"], l["up_proj"]], xs[2560], None, [ys["gate_proj"], ys["up_proj"]], workspace=kws[2560])
                        ql.linear_kq(l["down_proj"], xs[9728], out=ys["down_proj"], workspace=kws[9728])
                wall, ev = timed(graphed(kstep), 5, 2)
                nbytes = N_LAYERS * sum(n * (k // 256) * bb + M * k * 2 + M * n * 4 for n, k in shapes.values())
                kq["%s_m%d" % (kname, M)] = {"GBps": nbytes * 5 / wall / 1e9, "ms_per_step": wall / 5 * 1e3, "bytes_per_step": nbytes}
            x1 = torch.randn((1, 2560), device="cuda", generator=gen).to(torch.bfloat16)
            y1 = torch.empty((1, 9728), dtype=torch.float32, device="cuda")
            _, ev = timed(graphed(lambda: [ql.linear_kq(l["gate_proj"], x1, out=y1) for l in kpool]), 5, 2)
            per = ev / (5 * N_LAYERS)
            nb1 = 9728 * 10 * bb + 2560 * 2 + 9728 * 4
            kq["%s_m1" % kname]["gate_proj"] = {"us": per * 1e6, "GBps": nb1 / per / 1e9, "bytes": nb1}
            del kpool
            torch.cuda.empty_cache()
        extra["kquant_decode"] = kq
        # what a stream of launches of this size can reach at all: a read-only 16-byte streaming kernel over distinct buffers
        floor = {}
        big = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device="cuda", generator=gen)
        for nb_ in sorted({v["bytes"] for v in per_shape.values()} | {56199168}):
            n = nb_ // 16 * 16
            offs = [(i * 57000000) % ((1 << 30) - n) // 256 * 256 for i in range(40)]

            def fl():
                st = torch.cuda.current_stream().cuda_stream  # the capture stream while the graph is recorded
                for o in offs:
                    _lib.check(_lib.lib().mllm_hip_probe_copy(None, big.data_ptr() + o, n, st), "probe_copy")
            rp = graphed(fl)
            _, ev = timed(rp, 5, 2)
            floor[str(n)] = {"us": ev / (5 * 40) * 1e6, "GBps": n / (ev / (5 * 40)) / 1e9}
        del big
        extra["read_only_floor"] = floor
        # every launch shape against the read-only floor of its own byte count (1.0 = as fast as merely reading the bytes)
        extra["floor_over_launch"] = {name: round(floor[str(v["bytes"] // 16 * 16)]["us"] / v["us"], 3) for name, v in per_shape.items()}
        # the same GEMV kernel on a launch large enough to leave the fixed cost behind: gate + up of a Qwen3-32B-shaped layer
        # (2 x 25600 x 5120, 147 MB of Q4_0 blocks), eight distinct copies
        bigw = [[ql.PackedQWeight.synthetic(ql.Q4_0, 25600, 5120, gen) for _ in range(2)] for _ in range(8)]
        xb = torch.randn((1, 5120), device="cuda", generator=gen).to(torch.bfloat16)
        yb = [torch.empty((1, 25600), dtype=torch.float32, device="cuda") for _ in range(2)]
        _, ev = timed(graphed(lambda: [ql.linear_q_gemv_multi(ws, xb, None, ql.SCALE_X86_REF, yb) for ws in bigw]), 5, 2)
        per = ev / (5 * 8)
        nbig = 2 * synth.gemv_algorithmic_bytes(ql.Q4_0, 1, 25600, 5120, 2) - 5120 * 2
        # ... and with the activations handed over as the quantized image a producer kernel (RMSNorm) writes: no workgroup
        # quantizes (with 3200 workgroups the repeated quantization is what separates the two figures)
        _, imgb = ql.rmsnorm(xb.float(), torch.ones(5120, device="cuda"), 1e-6, want_image=True)
        _, ev2 = timed(graphed(lambda: [ql.linear_q_gemv_fused(ws, imgb, M=1, image=True, outs=yb) for ws in bigw]), 5, 2)
        per2 = ev2 / (5 * 8)
        extra["large_launch_gate_up_25600x5120"] = {"us": per * 1e6, "GBps": nbig / per / 1e9, "bytes": nbig,
                                                    "frac_of_hbm_peak": nbig / per / 1e9 / HBM_PEAK_GBS,
                                                    "from_quantized_image": {"us": per2 * 1e6, "GBps": nbig / per2 / 1e9,
                                                                             "frac_of_hbm_peak": nbig / per2 / 1e9 / HBM_PEAK_GBS}}
        del bigw
        # the Linear that ends every decode token of the model: lm_head, 151 936 x 2560 (mllm/models/qwen3/modeling_qwen3_fa2.hpp:264-265),
        # Q4_0, one row; four distinct copies (875 MB), one launch each, the kernel and launch shape the layer GEMVs take
        lmw = [ql.PackedQWeight.synthetic(ql.Q4_0, 151936, 2560, gen) for _ in range(4)]
        xl = torch.randn((1, 2560), device="cuda", generator=gen).to(torch.bfloat16)
        yl = torch.empty((1, 151936), dtype=torch.float32, device="cuda")
        _, ev = timed(graphed(lambda: [ql.linear_q_gemv(w, xl, None, ql.SCALE_X86_REF, out=yl) for w in lmw]), 5, 2)
        per = ev / (5 * 4)
        nlm = synth.gemv_algorithmic_bytes(ql.Q4_0, 1, 151936, 2560, 2)
        extra["lm_head_151936x2560"] = {"us": per * 1e6, "GBps": nlm / per / 1e9, "bytes": nlm,
                                        "frac_of_hbm_peak": nlm / per / 1e9 / HBM_PEAK_GBS}
        if wtype == ql.Q4_0 and args.m == 1:
            tok_s = head["ms_per_step"] * 1e-3 + per
            tok_b = head["bytes_per_step"] + nlm
            extra["decode_token_36_layers_plus_lm_head"] = {"ms": tok_s * 1e3, "GBps": tok_b / tok_s / 1e9, "bytes": tok_b,
                                                            "frac_of_hbm_peak": tok_b / tok_s / 1e9 / HBM_PEAK_GBS,
                                                            "note": "the measured step plus one lm_head launch (sum of the two times)"}
        del lmw
        extra["prefill_and_moe"] = side_workloads(torch, ql, synth, gen)

    cpu = None
    if not args.no_cpu:
        from oracle import oracle as orc
        rng = synth.rng_for(1)
        otype = orc.Q4_0 if wtype == ql.Q4_0 else orc.Q8_0
        Ws = {name: synth.make_weight(rng, otype, n, k) for name, (n, k) in shapes.items()}
        xsf = {k: synth.make_x_bf16(rng, args.m, k)[1] for k in (2560, 4096, 9728)}
        cores = len(os.sched_getaffinity(0))
        layer_bytes = step_bytes(wtype, args.m) / N_LAYERS

        def cpu_rate(threads, budget_s):
            """passes over one decoder layer with the AVX2 tile form of the reference's x86 path (tinyBLAS_Q0_AVX tiles, jobs
            split over `threads` as the op's threads option does), bit-identical to the scalar oracle"""
            for W in Ws.values():  # warm-up pass
                orc.linear_q_tiles(xsf[W.shape[1] * 32], W, otype, None, orc.SCALE_X86_REF, threads)
            passes, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < budget_s and passes < 400:
                for W in Ws.values():
                    orc.linear_q_tiles(xsf[W.shape[1] * 32], W, otype, None, orc.SCALE_X86_REF, threads)
                passes += 1
            return layer_bytes * passes / (time.perf_counter() - t0) / 1e9, passes
        v_all, p_all = cpu_rate(cores, 10.0)
        v_8, p_8 = cpu_rate(min(8, cores), 8.0)
        cpu = {"value": v_all, "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": "%d passes over ONE decoder layer (7 GEMVs, %.1f MB, M=%d) with the oracle's AVX2 tile form of the "
                         "reference's x86 path (quantize_row_q8_0 + tinyBLAS_Q0_AVX tiles with maddubs/madd block dots, jobs "
                         "split over the threads as llamafile_sgemm does), %d threads = every core this process may use; "
                         "bit-identical to the scalar oracle" % (p_all, layer_bytes / 1e6, args.m, cores),
               "at_reference_default_8_threads": {"value": v_8, "unit": "GB/s", "cores": min(8, cores), "passes": p_8}}

    out = {
        "metric": "W4 decode GEMV HBM GB/s" if wtype == ql.Q4_0 else "W8 decode GEMV HBM GB/s",
        "value": round(head["GBps"], 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Qwen3-4B decoder-layer decode GEMVs (q/k/v/o/gate/up/down), %s weights, bf16 x, M=%d; "
                               "one step = one decode token through 36 layers, %s, over %.2f GB of distinct weights"
                               % (args.wtype.upper(), args.m,
                                  "one launch per projection (252 launches)" if args.per_op else
                                  "sibling projections share a launch: qkv | o | gate+up | down (144 launches)",
                                  head["bytes_per_step"] / 1e9),
                   "M": args.m, "weights": args.wtype, "percent_of_hbm_peak": round(100 * head["GBps"] / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(dom["GBps"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom["GBps"] / HBM_PEAK_GBS, 4),
                     # FETCH_SIZE + WRITE_SIZE per dispatch from two rocprofv3 --pmc runs of `bench.py --pmc-probe`, each scaled
                     # by what the counter reads for the library's plain copy kernel of the same size
                     "traffic": traffic_from_profile() if (wtype == ql.Q4_0 and args.m == 1 and not args.per_op) else None,
                     "traffic_source": TRAFFIC_PROFILE if (wtype == ql.Q4_0 and args.m == 1 and not args.per_op) else None,
                     "kernel": ("gemv_q_kernel gate_proj N=9728 K=2560 M=%d" if args.per_op else
                                "gemv_q_kernel gate+up in one launch, 2 x (N=9728 K=2560), M=%d") % args.m, "us_per_launch": round(dom["us"], 3),
                     "algorithmic_bytes_per_launch": dom["bytes"]},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
