#!/usr/bin/env python3
"""Benchmark of the Q4 matmul path on one MI355X.

Headline workload (benchmark config 1): one Qwen3.5-2B-shaped decode layer at batch 1 —
Q4 GEMVs at hidden 2048: fused QKV (N=3072), O (N=2048), fused gate||up (N=12288, one
buffer and one launch, as the reference's decode does) and down (K=6144).  A "step" is
one layer: 4 GEMV launches over 30,146,560 bytes of Q4 blocks.  Steps rotate over
``--layers`` distinct weight sets (default 36 = 1.09 GB) so every launch streams its
weights from HBM rather than from the 256 MB Infinity Cache; the same loop over a single
layer gives the hot-cache figure reported beside it.

Prints ONE JSON line.  ``value`` = algorithmic bytes of all timed steps / wall time of the
timed region (HIP events on the launch stream, inputs resident in HBM).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense f16

# rocprofv3 counters on this workload (profiles/gemv_q4_b1_decode_layer_traffic.md): per layer step
# FETCH_SIZE 15122.0 KiB x 2.000 (copy-kernel scale) + WRITE_SIZE 144 KiB x 1.000, over 4 launches
MEASURED_TRAFFIC_PER_LAUNCH = (15122.0 * 2.0 + 144.0) * 1024 / 4
# The same counters on the prefill GEMM of config 2 at M = 2048, N = 17408, K = 5120 (same file): gemm_q4_w2 and its
# pack pass fetch 797.1 + 21.0 MB and write 242.5 + 21.0 MB per call, against 76.7 + 21.0 MB read and 142.6 MB written
# algorithmically (the packed activations are re-read per XCD and group of weight-tile columns, out of the
# Infinity Cache; K-sliced tail tiles write partial sums)
MEASURED_GEMM_TRAFFIC_PER_LAUNCH = (797.1 + 21.0 + 242.5 + 21.0) * 1e6

LAYER = [("qkv", 3072, 2048), ("o", 2048, 2048), ("gate_up", 12288, 2048), ("down", 2048, 6144)]


def gemv_bytes(n, k, batch):
    """Algorithmic bytes of one GEMV launch: Q4 blocks + x read + y written."""
    return n * (k // 32) * 20 + batch * k * 4 + batch * n * 4


def device_q4_weight(torch, n, k, gen):
    """Synthetic native-layout blocks generated on the device (same distribution as
    lattice_amd.synth.q4_weight: scale |N(0,0.02)|/7 as f16, bias -8*scale, uniform nibbles)."""
    nb = n * (k // 32)
    s = (torch.randn(nb, device="cuda", generator=gen).abs() * (0.02 / 7.0)).clamp_min(6.2e-5)
    blocks = torch.empty((nb, 20), dtype=torch.uint8, device="cuda")
    blocks[:, 0:2] = s.to(torch.float16).view(torch.uint8).view(nb, 2)
    blocks[:, 2:4] = (-8.0 * s).to(torch.float16).view(torch.uint8).view(nb, 2)
    blocks[:, 4:] = torch.randint(0, 256, (nb, 16), dtype=torch.uint8, device="cuda", generator=gen)
    return blocks.view(-1)


def device_q8_weight(torch, n, k, gen):
    """Synthetic Q8_0 blocks generated on the device: f16 scale |N(0,0.02)|/127, uniform int8."""
    nb = n * (k // 32)
    s = (torch.randn(nb, device="cuda", generator=gen).abs() * (0.02 / 127.0)).clamp_min(6.2e-5)
    blocks = torch.empty((nb, 34), dtype=torch.uint8, device="cuda")
    blocks[:, 0:2] = s.to(torch.float16).view(torch.uint8).view(nb, 2)
    blocks[:, 2:] = torch.randint(1, 256, (nb, 32), dtype=torch.uint8, device="cuda", generator=gen)
    blocks[:, 2:][blocks[:, 2:] == 128] = 129  # -128 is never produced by the quantiser
    return blocks.view(-1)


def device_q3_weight(torch, n, k, gen):
    """Synthetic Q3 blocks generated on the device: f16 scale |N(0,0.02)|/3.5, bias -4*scale,
    uniform plane bits."""
    nb = n * (k // 32)
    s = (torch.randn(nb, device="cuda", generator=gen).abs() * (0.02 / 3.5)).clamp_min(6.2e-5)
    blocks = torch.empty((nb, 16), dtype=torch.uint8, device="cuda")
    blocks[:, 0:2] = s.to(torch.float16).view(torch.uint8).view(nb, 2)
    blocks[:, 2:4] = (-4.0 * s).to(torch.float16).view(torch.uint8).view(nb, 2)
    blocks[:, 4:] = torch.randint(0, 256, (nb, 12), dtype=torch.uint8, device="cuda", generator=gen)
    return blocks.view(-1)


def timed(torch, fn, iters):
    """Average milliseconds per call of fn over `iters` back-to-back calls (HIP events on the
    current stream, which is the stream every launch goes to)."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(iters):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


MIN_TIMED_MS = 20.0  # every graph-timed figure covers at least this much GPU time
LAST_TIMING = {}


def graph_timed(torch, fn, iters, replays=3):
    """Like timed(), but the `iters` calls are captured once into a HIP graph and the graph is
    replayed: the launches reach the GPU back to back, with no per-call host overhead between
    them.  The graph is replayed at least `replays` times and as often as it takes to cover
    MIN_TIMED_MS of GPU time, each replay between its own pair of HIP events.  Returns the MEAN
    milliseconds per call over all timed replays; the minimum and the replay count are left in
    LAST_TIMING."""
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        for i in range(iters):
            fn(i)
    torch.cuda.synchronize()
    g.replay()  # untimed: first replay of a fresh graph
    per_replay = []
    while len(per_replay) < replays or (sum(per_replay) < MIN_TIMED_MS and len(per_replay) < 2000):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        g.replay()
        stop.record()
        torch.cuda.synchronize()
        per_replay.append(start.elapsed_time(stop))
    del g
    LAST_TIMING.clear()
    LAST_TIMING.update(mean_ms=sum(per_replay) / len(per_replay) / iters, min_ms=min(per_replay) / iters,
                       replays=len(per_replay), timed_region_ms=sum(per_replay))
    return LAST_TIMING["mean_ms"]


def read_sweep(torch, be):
    """Read-bandwidth ceiling of this GPU by launch size: the read probe over a 4 GB pool (launch i
    reads piece i, so nothing is served from a cache), swept over grid, bytes in flight per thread,
    chunked or interleaved workgroups and plain or non-temporal loads.  Prints a table."""
    pool_bytes = 4 << 30
    pool = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
    pool.fill_(1)
    sizes = [7864320, 30146560, 55705600, 318767104, 1 << 30]
    print("%-22s %12s %6s %9s %9s" % ("variant", "bytes", "grid", "us", "GB/s"))
    for sz in sizes:
        best = None
        for strided in (False, True):
            for nt in (False, True):
                for fl in (64, 128, 256):
                    for grid in (256, 512, 1024, 2048, 4096, 8192):
                        nbuf = min(200, pool_bytes // sz)
                        iters = 12 if sz > (100 << 20) else 100
                        f = lambda i: be.probe_read_config(pool, sz, grid, fl, strided, nt, offset=(i % nbuf) * sz)
                        f(0)
                        ms = graph_timed(torch, f, iters, replays=2)
                        name = "%s %3dB%s" % ("interleaved" if strided else "chunked", fl, " nt" if nt else "")
                        print("%-22s %12d %6d %9.2f %9.1f" % (name, sz, grid, ms * 1e3, sz / ms / 1e6), flush=True)
                        if best is None or ms < best[0]:
                            best = (ms, name, grid)
        print("best at %d bytes: %s grid %d: %.2f us = %.1f GB/s" % (sz, best[1], best[2], best[0] * 1e3, sz / best[0] / 1e6),
              flush=True)


def prefill_gemm(torch, be, gen, tm):
    """BASELINE config 2: the 27B MLP matrices at 512 and 2048 tokens, f16 activations."""
    gemm = {}
    for (n, k) in ((17408, 5120), (5120, 17408)):
        qw = be.wrap_device_blocks(device_q4_weight(torch, n, k, gen))
        for m in (512, 2048):
            x = torch.randn((m, k), device="cuda", generator=gen).to(torch.float16)
            y = torch.empty((m, n), device="cuda")
            f = lambda i: be.dispatch_gemm(x, 0, qw, y, 0, m, n, k)
            for i in range(3):
                f(i)
            ms = tm(torch, f, 10)
            tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
            gemm["M%d_N%d_K%d" % (m, n, k)] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 1),
                                               "pct_of_f16_mfma_peak": round(100 * tf / MFMA_F16_PEAK_TFLOPS, 2)}
        del qw
    return gemm


def moe_section(torch, be, gen, tm, synth):
    """BASELINE config 4 (grouped expert GEMV), the whole MoE layer in its call forms, and the one-token layer."""
    out = {}
    # MoE grouped expert GEMV, benchmark config 4
    mo = synth.MOE_35B
    E, I, H, T, TK = mo["experts"], mo["inter"], mo["hidden"], mo["tokens"], mo["top_k"]
    sets = []
    for _ in range(10):  # 10 x 125.8 MB of expert tensors
        sets.append((be.wrap_device_blocks(device_q4_weight(torch, E * 2 * I, H, gen)),
                     be.wrap_device_blocks(device_q4_weight(torch, E * H, I, gen))))
    lg = torch.from_numpy(synth.router_logits(T, E, seed=0)).cuda()
    ids, wts = be.moe_route(lg, TK)
    xm = torch.randn((T, H), device="cuda", generator=gen)
    ym = torch.empty((T, H), device="cuda")
    distinct = int(torch.unique(ids).numel())
    moe_bytes = distinct * (2 * I * (H // 32) * 20 + H * (I // 32) * 20) + 2 * T * H * 4
    f = lambda i: be.moe_experts(sets[i % len(sets)][0], sets[i % len(sets)][1], E, I, H, xm, ids, wts, ym)
    for i in range(len(sets)):
        f(i)
    ms = tm(torch, f, 40)
    # the same step with the router in front of it (softmax, top-k, renormalise from the logits)
    def routed(i):
        ids_i, wts_i = be.moe_route(lg, TK)
        be.moe_experts(sets[i % len(sets)][0], sets[i % len(sets)][1], E, I, H, xm, ids_i, wts_i, ym)
    for i in range(3):
        routed(i)
    ms_routed = tm(torch, routed, 40)
    # ... and with the always-active shared expert (same intermediate size) added onto the sum
    shared = [(be.wrap_device_blocks(device_q4_weight(torch, 2 * I, H, gen)),
               be.wrap_device_blocks(device_q4_weight(torch, H, I, gen))) for _ in range(len(sets))]
    sgate = torch.randn((H,), device="cuda", generator=gen) * (1.0 / H ** 0.5)
    def whole_layer(i):
        routed(i)
        sh = shared[i % len(shared)]
        be.moe_shared_expert(sh[0], sh[1], sgate, I, H, xm, ym)
    for i in range(3):
        whole_layer(i)
    ms_layer = tm(torch, whole_layer, 40)
    # ... and as one call (lq4_moe_ffn)
    def one_call(i):
        sh = shared[i % len(shared)]
        be.moe_ffn(lg, sets[i % len(sets)][0], sets[i % len(sets)][1], E, TK, I, sh[0], sh[1], sgate, I, H, xm, ym)
    for i in range(3):
        one_call(i)
    ms_one = tm(torch, one_call, 40)
    # decode: the same layer for one token (8 routed experts + the shared one, 28.3 MB)
    lg1, x1, y1 = lg[:1].contiguous(), xm[:1].contiguous(), torch.empty((1, H), device="cuda")
    def decode_layer(i):
        sh = shared[i % len(shared)]
        be.moe_ffn(lg1, sets[i % len(sets)][0], sets[i % len(sets)][1], E, TK, I, sh[0], sh[1], sgate, I, H, x1, y1)
    for i in range(3):
        decode_layer(i)
    ms_decode = tm(torch, decode_layer, 40)
    decode_bytes = (TK + 1) * (2 * I * (H // 32) * 20 + H * (I // 32) * 20)
    out["moe_layer_one_token"] = {"algorithmic_bytes": decode_bytes, "ms_per_step": round(ms_decode, 4),
                                  "GB/s": round(decode_bytes / ms_decode / 1e6, 1),
                                  "pct_of_hbm_peak": round(100 * decode_bytes / ms_decode / 1e6 / HBM_PEAK_GBPS, 2),
                                  "launches": 2}
    out["moe_grouped_gemv"] = {"distinct_experts": distinct, "algorithmic_bytes": moe_bytes,
                               "ms_per_step": round(ms, 4), "GB/s": round(moe_bytes / ms / 1e6, 1),
                               "pct_of_hbm_peak": round(100 * moe_bytes / ms / 1e6 / HBM_PEAK_GBPS, 2),
                               "ms_per_step_with_router": round(ms_routed, 4),
                               "ms_per_step_with_router_and_shared_expert": round(ms_layer, 4),
                               "ms_per_step_whole_layer_one_call": round(ms_one, 4)}
    del sets, shared
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=720)
    ap.add_argument("--warmup", type=int, default=72)
    ap.add_argument("--layers", type=int, default=36, help="distinct weight sets to rotate over")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--skip-extras", action="store_true", help="headline workload only")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="run nothing but warmup and the timed headline region (for kernel-trace profiles)")
    ap.add_argument("--gemm-only", action="store_true",
                    help="run the four config-2 prefill GEMM shapes and nothing else (for counter runs)")
    ap.add_argument("--moe-only", action="store_true",
                    help="only the MoE lines (config 4, whole layer, one-token layer): for profiling")
    ap.add_argument("--read-sweep", action="store_true",
                    help="print the read-probe sweep (grid x bytes in flight x access pattern x size) and exit")
    ap.add_argument("--eager", action="store_true",
                    help="launch every step from Python instead of replaying a captured HIP graph")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path is measured on one GPU only (one process, one device); "
                 "run with --gpus 1")

    import torch
    from lattice_amd import backend, synth

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    be = backend.HipQ4Backend(0)
    if args.read_sweep:
        read_sweep(torch, be)
        return
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    B = args.batch
    if args.gemm_only:
        print(json.dumps({"prefill_gemm_f16": prefill_gemm(torch, be, gen, graph_timed)}))
        return
    if args.moe_only:
        print(json.dumps(moe_section(torch, be, gen, graph_timed, synth)))
        return

    # ---- resident inputs ------------------------------------------------------------
    layers = []
    for li in range(args.layers):
        bufs = {}
        for name, n, k in LAYER:
            t = device_q4_weight(torch, n, k, gen)
            bufs[name] = be.wrap_device_blocks(t)
        layers.append(bufs)
    xs = {k: torch.randn((B, k), device="cuda", generator=gen) for k in (2048, 6144)}
    ys = {n: torch.empty((B, n), device="cuda") for _, n, _ in LAYER}
    step_bytes = sum(gemv_bytes(n, k, B) for _, n, k in LAYER)
    weight_bytes = sum(n * (k // 32) * 20 for _, n, k in LAYER)

    def layer_step(i, pool=layers):
        bufs = pool[i % len(pool)]
        for name, n, k in LAYER:
            be.gemv_batch(xs[k], bufs[name], ys[n], B, n, k)

    # ---- correctness spot check against the oracle on this run's own buffers ---------
    check = {}
    try:
        import oracle
        name, n, k = LAYER[1]
        ychk = torch.empty((B, n), device="cuda")
        be.gemv_batch(xs[k], layers[0][name], ychk, B, n, k)
        wq = layers[0][name]._keepalive.cpu().numpy()
        ref = oracle.gemm_f32(xs[k].cpu().numpy(), wq, n, k)
        got = ychk.cpu().numpy()
        check = {"shape": [n, k], "rel_err_vs_oracle": float(np.abs(got - ref).max() / np.abs(ref).max())}
        assert check["rel_err_vs_oracle"] <= 1e-3, check
    except ImportError:
        check = {"skipped": "oracle not importable"}

    # ---- headline: rotating (HBM) ------------------------------------------------------
    for i in range(args.warmup):
        layer_step(i)
    tm = timed if args.eager else graph_timed
    ms_step = tm(torch, layer_step, args.steps)
    headline_timing = dict(LAST_TIMING) if not args.eager else {}
    if args.headline_only:
        args.skip_extras = args.skip_cpu = True
    eager_ms = ms_step if args.headline_only else timed(torch, layer_step, args.steps)
    value = step_bytes / (ms_step * 1e-3) / 1e9
    launches_per_step = len(LAYER)
    us_per_launch = ms_step * 1e3 / launches_per_step

    # same loop on one layer: weights stay in the Infinity Cache
    hot_ms = ms_step if args.headline_only else tm(torch, lambda i: layer_step(0), max(50, args.steps // 4))

    out = {
        "metric": "Q4 GEMV HBM GB/s @batch 1 (Qwen3.5-2B decode layer)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u4 weights x f32 activations, f32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE config 1: Qwen3.5-2B-shaped decode layer, batch %d: qkv(3072x2048) + "
                        "o(2048x2048) + fused gate||up(12288x2048) + down(2048x6144), Q4 group 32" % B,
            "batch": B,
            "launches_per_step": launches_per_step,
            "distinct_layers_rotated": args.layers,
            "rotating_weight_bytes": weight_bytes * args.layers,
            "algorithmic_bytes_per_step": step_bytes,
        },
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "tokens_per_s_equivalent_24_layers": round(1.0 / (24 * ms_step * 1e-3), 1),
        "launch_mode": "eager launches from Python" if args.eager else "captured HIP graph, replayed",
        "timing": {"value_is": "mean over replays", "replays": headline_timing.get("replays"),
                   "timed_region_ms": round(headline_timing.get("timed_region_ms", 0.0), 3),
                   "ms_per_step_min_over_replays": round(headline_timing.get("min_ms", ms_step), 5)},
        "eager_python_launch": {"ms_per_step": round(eager_ms, 5),
                                "GB/s": round(step_bytes / (eager_ms * 1e-3) / 1e9, 1)},
        "hot_cache": {"ms_per_step": round(hot_ms, 5),
                      "GB/s": round(step_bytes / (hot_ms * 1e-3) / 1e9, 1)},
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_q4_b1" if B == 1 else "gemv_q4_mfma",
            "achieved": round(value, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(value / HBM_PEAK_GBPS, 4),
            # HBM-side bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what
            # the same counter reads for the library's plain copy kernel; measured on this workload
            "traffic": MEASURED_TRAFFIC_PER_LAUNCH if B == 1 else None,
            "algorithmic_bytes_per_launch": step_bytes / launches_per_step,
            "avg_launch_us": round(us_per_launch, 3),
        },
        "parity_check": check,
    }

    # ---- per-shape and secondary workloads ---------------------------------------------
    if not args.skip_extras:
        # Per shape: the GEMV and, on the same buffers, the read-only probe kernel whose time is
        # the ceiling for a launch of that size on this GPU.  "27b_*" are the benchmark config 2
        # matrices driven as batch-1 decode GEMVs: launches large enough to approach the HBM
        # streaming rate.
        shapes = {}
        # "lm_head" is the reference's largest single GEMV per token (vocabulary 248,320 x hidden 2048,
        # 318 MB of Q4 blocks): one launch big enough to show the kernel's streaming rate; "27b_lm_head" the same
        # projection at the 27B-shaped hidden size of config 2 (151,936 x 5120, 486 MB).
        extra_shapes = [("cfg0", 4096, 1024), ("27b_up", 17408, 5120), ("27b_down", 5120, 17408),
                        ("lm_head", 248320, 2048), ("27b_lm_head", 151936, 5120)]
        for name, n, k in LAYER + extra_shapes:
            wbytes = n * (k // 32) * 20
            pool = [l[name] for l in layers] if name in dict((a, 1) for a, _, _ in LAYER) else \
                [be.wrap_device_blocks(device_q4_weight(torch, n, k, gen))
                 for _ in range(max(3, min(400, int(1.2e9 // wbytes))))]
            x = torch.randn((B, k), device="cuda", generator=gen)
            y = torch.empty((B, n), device="cuda")
            f = lambda i, pool=pool, x=x, y=y, n=n, k=k: be.gemv_batch(x, pool[i % len(pool)], y, B, n, k)
            pr = lambda i, pool=pool: be.probe_read(pool[i % len(pool)]._keepalive)
            for i in range(len(pool)):
                f(i)
            reps = max(4 * len(pool), 100) if wbytes < 3e7 else 2 * len(pool)
            # (the first timed pass over a freshly built pool runs 5-7 % slow on the large matrices -- the GPU has
            # idled through the pool's generation and the capture -- while the probe, timed later, does not: one
            # pass is timed and dropped, so that the GEMV and its probe are measured in the same state)
            tm(torch, f, reps)
            cold = tm(torch, f, reps)
            hot = tm(torch, lambda i: f(0), 100)
            pcold = tm(torch, pr, reps)
            by = gemv_bytes(n, k, B)
            shapes[name] = {"n": n, "k": k, "bytes": by, "cold_us": round(cold * 1e3, 3),
                            "cold_GB/s": round(by / cold / 1e6, 1), "hot_us": round(hot * 1e3, 3),
                            "hot_GB/s": round(by / hot / 1e6, 1),
                            "read_probe_cold_us": round(pcold * 1e3, 3),
                            "read_probe_cold_GB/s": round(wbytes / pcold / 1e6, 1),
                            "gemv_vs_probe": round(pcold / cold, 3)}
            if name == "lm_head" and B == 1:
                # the same projection with the exact top-50 selection behind it (fused lm_head + top-k)
                ftk = lambda i, pool=pool, x=x, n=n, k=k: be.lm_head_topk(x, pool[i % len(pool)], n, k, 50)
                for i in range(len(pool)):
                    ftk(i)
                tk = tm(torch, ftk, reps)
                shapes[name]["with_top50_us"] = round(tk * 1e3, 3)
                shapes[name]["with_top50_GB/s"] = round(by / tk / 1e6, 1)
            del pool
        out["gemv_shapes_batch%d" % B] = shapes

        # sibling formats, batch 1: the MLP matrices of the decode layer and the lm_head
        if B == 1:
            for fmt, block_bytes, make, call in (("q8_0", 34, device_q8_weight, be.dispatch_matmul_q8),
                                                 ("q3", 16, device_q3_weight, be.dispatch_matmul_q3)):
                res = {}
                for name, n, k in [("gate_up", 12288, 2048), ("down", 2048, 6144), ("27b_up", 17408, 5120),
                                   ("lm_head", 248320, 2048)]:
                    wbytes = n * (k // 32) * block_bytes
                    pool = [be.wrap_device_blocks(make(torch, n, k, gen))
                            for _ in range(max(2, min(200, int(1.1e9 // wbytes))))]
                    x = torch.randn((1, k), device="cuda", generator=gen)
                    y = torch.empty((1, n), device="cuda")
                    f = lambda i, pool=pool, x=x, y=y, n=n, k=k, call=call: call(x, pool[i % len(pool)], y, 1, n, k)
                    pr = lambda i, pool=pool: be.probe_read(
                        pool[i % len(pool)]._keepalive[:len(pool[0]._keepalive) // 16 * 16])
                    for i in range(len(pool)):
                        f(i)
                    reps = max(4 * len(pool), 100) if wbytes < 3e7 else 2 * len(pool)
                    cold, pcold = tm(torch, f, reps), tm(torch, pr, reps)
                    by = wbytes + 4 * k + 4 * n
                    res[name] = {"n": n, "k": k, "bytes": by, "cold_us": round(cold * 1e3, 3),
                                 "cold_GB/s": round(by / cold / 1e6, 1),
                                 "read_probe_cold_us": round(pcold * 1e3, 3), "gemv_vs_probe": round(pcold / cold, 3)}
                    del pool
                out[fmt + "_gemv_batch1"] = res

        if B == 1:
            x8 = {k: torch.randn((8, k), device="cuda", generator=gen) for k in (2048, 6144)}
            y8 = {n: torch.empty((8, n), device="cuda") for _, n, _ in LAYER}

            def step8(i):
                bufs = layers[i % len(layers)]
                for name, n, k in LAYER:
                    be.gemv_batch(x8[k], bufs[name], y8[n], 8, n, k)
            for i in range(len(layers)):
                step8(i)
            ms8 = tm(torch, step8, max(72, args.steps // 2))
            b8 = sum(gemv_bytes(n, k, 8) for _, n, k in LAYER)
            out["decode_layer_batch8"] = {"ms_per_step": round(ms8, 5), "GB/s": round(b8 / ms8 / 1e6, 1),
                                          "pct_of_hbm_peak": round(100 * b8 / ms8 / 1e6 / HBM_PEAK_GBPS, 2)}

        # The same four matrices as the real dependent chain of a token (o -> +residual, RMSNorm -> gate||up
        # -> silu*up -> down -> +residual, RMSNorm -> qkv) through lq4_gemv_chain (one fused launch per step).
        if B == 1:
            cres, cres1, cres2 = (torch.randn(2048, device="cuda", generator=gen) for _ in range(3))
            cg1, cg2 = (0.1 * torch.randn(2048, device="cuda", generator=gen) for _ in range(2))
            cqkv = torch.empty(3072, device="cuda")
            chains = [[
                be.chain_step(b["o"], 2048, 2048, x=xs[2048][0]),
                be.chain_step(b["gate_up"], 12288, 2048, from_previous=True, norm=(cres, None, cg1, 1e-6, cres1),
                              silu_mul_pairs=True),
                be.chain_step(b["down"], 2048, 6144, from_previous=True),
                be.chain_step(b["qkv"], 3072, 2048, from_previous=True, norm=(cres1, None, cg2, 1e-6, cres2), y=cqkv)]
                for b in layers]
            cf = lambda i: be.dispatch_chain(chains[i % len(chains)])
            for i in range(len(layers)):
                cf(i)
            be.synchronize()
            ms_c = tm(torch, cf, max(72, args.steps // 2))
            be.synchronize()
            ch = {"us_per_step": round(ms_c * 1e3, 3), "GB/s": round(step_bytes / ms_c / 1e6, 1),
                  "pct_of_hbm_peak": round(100 * step_bytes / ms_c / 1e6 / HBM_PEAK_GBPS, 2)}
            ch["note"] = ("dependent chain incl. residual adds, RMSNorms and silu*up; the headline's four GEMVs "
                          "alone are independent launches over the same weights")
            out["decode_layer_chain"] = ch

        # decode MLP with its elementwise neighbours: residual add + RMSNorm, gate||up GEMV, silu*up,
        # down GEMV, add into the residual.  Five launches one by one against two fused launches.
        if B == 1:
            hid, inter = 2048, 6144
            gamma_v = torch.randn(hid, device="cuda", generator=gen) * 0.1
            for rows in (1, 8):  # one token, and the decode steps of eight sequences at once
                base_v = torch.randn((rows, hid), device="cuda", generator=gen)
                delta_v = torch.randn((rows, hid), device="cuda", generator=gen)
                res_v, normed_v, hid_v, ffn_v = (torch.empty((rows, hid), device="cuda") for _ in range(4))
                gu_v, act_v = torch.empty((rows, 2 * inter), device="cuda"), torch.empty((rows, inter), device="cuda")

                def mlp_unfused(i, rows=rows):
                    bufs = layers[i % len(layers)]
                    be.dispatch_fused_residual_add_norm(base_v, delta_v, res_v, normed_v, gamma_v, hid, 1e-6, num_rows=rows)
                    be.gemv_batch(normed_v, bufs["gate_up"], gu_v, rows, 2 * inter, hid)
                    be.dispatch_silu_mul_fused(gu_v, inter, rows, out=act_v, out_stride=inter)
                    be.gemv_batch(act_v, bufs["down"], ffn_v, rows, hid, inter)
                    be.dispatch_add_and_copy(ffn_v, res_v, hid_v, rows * hid)

                def mlp_fused(i, rows=rows):
                    bufs = layers[i % len(layers)]
                    be.dispatch_matmul_fused(None, bufs["gate_up"], gu_v, 2 * inter, hid,
                                             norm=(base_v, delta_v, gamma_v, 1e-6, res_v), batch=rows)
                    be.dispatch_matmul_fused(gu_v, bufs["down"], None, hid, inter, silu_mul=True,
                                             add_residual=(res_v, hid_v), batch=rows)

                def mlp_fused_pairs(i):  # one row: silu(gate) * up formed by the first launch
                    bufs = layers[i % len(layers)]
                    be.dispatch_matmul_fused(None, bufs["gate_up"], act_v, 2 * inter, hid,
                                             norm=(base_v, delta_v, gamma_v, 1e-6, res_v), silu_mul_pairs=True)
                    be.dispatch_matmul_fused(act_v, bufs["down"], None, hid, inter, add_residual=(res_v, hid_v))
                mlp = {}
                forms = [("five_launches", mlp_unfused), ("two_fused_launches_silu_in_second", mlp_fused)]
                forms.append(("two_fused_launches", mlp_fused_pairs) if rows == 1 else ("two_fused_launches", mlp_fused))
                for nm, f in forms:
                    for i in range(len(layers)):
                        f(i)
                    mlp[nm + "_us"] = round(tm(torch, f, max(72, args.steps // 2)) * 1e3, 3)
                mlp_bytes = gemv_bytes(2 * inter, hid, rows) + gemv_bytes(hid, inter, rows)
                mlp["GB/s_fused"] = round(mlp_bytes / mlp["two_fused_launches_us"] / 1e3, 1)
                mlp["speedup"] = round(mlp["five_launches_us"] / mlp["two_fused_launches_us"], 3)
                out["decode_mlp_hidden2048_inter6144" + ("" if rows == 1 else "_rows%d" % rows)] = mlp

        # single-LoRA epilogue, benchmark config 3: q (2048x2048) and v (512x2048) projections, rank 16,
        # f16 factors, scale alpha/r = 2.0, fused into the projection's own launch
        if B == 1:
            from lattice_amd import synth
            r = 16
            projs = [("q_proj", 2048, 2048), ("v_proj", 512, 2048)]
            pool = [{nm: be.wrap_device_blocks(device_q4_weight(torch, n, k, gen)) for nm, n, k in projs}
                    for _ in range(96)]  # 315 MB: more than the Infinity Cache
            mods = {nm: synth.lora_pair(r, k, n, seed=0, tag=nm) for nm, n, k in projs}
            lora_out = {}
            for bsz in (1, 8, 64):
                xl = torch.randn((bsz, 2048), device="cuda", generator=gen)
                yl = {nm: torch.empty((bsz, n), device="cuda") for nm, n, _ in projs}

                def lstep(i, use_lora, bsz=bsz, xl=xl, yl=yl):
                    bufs = pool[i % len(pool)]
                    for nm, n, k in projs:
                        kw = dict(layer_idx=0, module=nm) if use_lora else {}
                        if bsz <= 16:
                            be.gemv_batch(xl, bufs[nm], yl[nm], bsz, n, k, **kw)
                        else:
                            be.dispatch_gemm(xl, 0, bufs[nm], yl[nm], 0, bsz, n, k, **kw)
                res = {}
                for use_lora in (False, True):
                    if use_lora:
                        be.load_lora_adapter([backend.LoraLayerData(0, mods)], scale=32 / r)
                    f = lambda i, u=use_lora: lstep(i, u)
                    for i in range(len(pool)):
                        f(i)
                    res[use_lora] = tm(torch, f, 192)
                    if use_lora:
                        be.unload_lora_adapter()
                lb = sum(gemv_bytes(n, k, bsz) + 2 * r * (k + n) + bsz * r * 4 for _, n, k in projs)
                lora_out["batch%d" % bsz] = {"base_us": round(res[False] * 1e3, 3),
                                             "with_lora_us": round(res[True] * 1e3, 3),
                                             "GB/s_with_lora": round(lb / res[True] / 1e6, 1),
                                             "lora_overhead_pct": round(100 * (res[True] / res[False] - 1), 1)}
                if bsz <= 128:
                    # the same two projections through lq4_gemv_multi: one call for both (one launch at batch 1,
                    # every adapter's A . x in one more up to 16 rows; above, one packed image of x for both)
                    def mstep(i, use_lora, bsz=bsz, xl=xl, yl=yl):
                        bufs = pool[i % len(pool)]
                        be.gemv_multi(xl, [(bufs[nm], n, yl[nm], nm) for nm, n, _ in projs], bsz, 2048,
                                      layer_idx=0 if use_lora else None)
                    mres = {}
                    for use_lora in (False, True):
                        if use_lora:
                            be.load_lora_adapter([backend.LoraLayerData(0, mods)], scale=32 / r)
                        f = lambda i, u=use_lora: mstep(i, u)
                        for i in range(len(pool)):
                            f(i)
                        mres[use_lora] = tm(torch, f, 192)
                        if use_lora:
                            be.unload_lora_adapter()
                    lora_out["batch%d" % bsz].update({
                        "one_call_base_us": round(mres[False] * 1e3, 3),
                        "one_call_with_lora_us": round(mres[True] * 1e3, 3),
                        "one_call_GB/s_with_lora": round(lb / mres[True] / 1e6, 1),
                        "one_call_lora_overhead_pct": round(100 * (mres[True] / mres[False] - 1), 1)})
            out["lora_q_v_rank16"] = lora_out
            del pool

        # prefill GEMM, benchmark config 2
        del layers
        torch.cuda.empty_cache()
        gemm = prefill_gemm(torch, be, gen, tm)
        out["prefill_gemm_f16"] = gemm
        # the GEMM half of the metric as a roofline object of its own: the largest config-2 problem
        big = gemm["M2048_N17408_K5120"]
        out["roofline_gemm"] = {
            "bound": "mfma", "kernel": "gemm_q4 (prefill)", "workload": "BASELINE config 2: M=2048, N=17408, K=5120",
            "achieved": big["TFLOP/s"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(big["TFLOP/s"] / MFMA_F16_PEAK_TFLOPS, 4),
            "flops_per_launch": 2.0 * 2048 * 17408 * 5120, "avg_launch_us": round(big["ms"] * 1e3, 2),
            "traffic": MEASURED_GEMM_TRAFFIC_PER_LAUNCH,
            "other_shapes_frac": {k_: round(v_["TFLOP/s"] / MFMA_F16_PEAK_TFLOPS, 4) for k_, v_ in gemm.items()},
        }

        # the same for the sibling formats (one shape each way), and their few-token kernel at 16 rows
        sib = {}
        for fmt, make, call in (("q8_0", device_q8_weight, be.dispatch_gemm_q8),
                                ("q3", device_q3_weight, be.dispatch_gemm_q3)):
            res = {}
            for (n, k) in ((17408, 5120), (5120, 17408)):
                qw = be.wrap_device_blocks(make(torch, n, k, gen))
                for m in (16, 2048):
                    x = torch.randn((m, k), device="cuda", generator=gen).to(torch.float16)
                    y = torch.empty((m, n), device="cuda")
                    f = lambda i: call(x, 0, qw, y, 0, m, n, k)
                    for i in range(3):
                        f(i)
                    ms = tm(torch, f, 10)
                    res["M%d_N%d_K%d" % (m, n, k)] = {"ms": round(ms, 4),
                                                      "TFLOP/s": round(2.0 * m * n * k / (ms * 1e-3) / 1e12, 1)}
                del qw
            sib[fmt] = res
        out["sibling_gemm_f16"] = sib

        out.update(moe_section(torch, be, gen, tm, synth))

        # plain copies of known size: what a profiler's HBM traffic counters are scaled by
        csrc = torch.empty(64 << 20, dtype=torch.int32, device="cuda").random_(generator=gen)
        cdst = torch.empty_like(csrc)
        for _ in range(3):
            be.probe_copy(csrc, cdst)
        torch.cuda.synchronize()
        out["traffic_calibration"] = {"kernel": "probe_copy_kernel", "bytes_read": csrc.numel() * 4,
                                      "bytes_written": csrc.numel() * 4, "launches": 3}
        del csrc, cdst

    # ---- CPU baseline: the reference's CPU route, timed on this box's host cores --------
    if not args.skip_cpu:
        import oracle
        cpu_layer = [(n, k, synth.q4_weight(n, k, seed=0, tag=name)) for name, n, k in LAYER]
        cpu_x = {k: synth.activations(B, k, seed=0) for k in (2048, 6144)}
        scratch = np.zeros(max(n * k for n, k, _ in cpu_layer), dtype=np.float32)
        res = {}
        for mode, label in ((0, "reference_dispatch"), (1, "forced_avx2_dot")):
            t0 = time.perf_counter()
            reps = 0
            kid = None
            while True:
                for n, k, wq in cpu_layer:
                    _, kid = oracle.cpu_q4_matmul(cpu_x[k], wq, scratch, B, n, k, mode=mode)
                reps += 1
                el = time.perf_counter() - t0
                if el > (8.0 if mode == 0 else 4.0) or reps >= 200:
                    break
            res[label] = {"s_per_layer": el / reps, "GB/s_over_q4_bytes": step_bytes * reps / el / 1e9,
                          "reps": reps, "matmul_kernel": oracle.KERNEL_NAMES[kid]}
        out["cpu_baseline"] = {
            "value": round(res["reference_dispatch"]["GB/s_over_q4_bytes"], 4),
            "unit": "GB/s",
            "cores": 1,
            "kind": "port",
            "sample": "%d passes of the same decode layer (4 Q4 matrices, batch %d): dequantize_row_q4_0 "
                      "to f32 then matmul_bt with the reference's non-macOS dispatch, single thread (the "
                      "reference CPU matmul is single-threaded); host has %d cores"
                      % (res["reference_dispatch"]["reps"], B, os.cpu_count()),
            "matmul_kernel": res["reference_dispatch"]["matmul_kernel"],
            "forced_avx2_dot_GB/s": round(res["forced_avx2_dot"]["GB/s_over_q4_bytes"], 4),
        }

    out["path_counters"] = be.path_counters()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
