#!/usr/bin/env python3
"""Benchmark of the quantized MoE block on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the MoE block over one batch: 3 tokens (three concurrent sequences, one token
each), 256 experts top-8 + 1 shared, hidden 2048, expert width 512, Q6_K experts, Q8_0 router and
shared expert -- BASELINE.json configs[1].  Successive steps run on different, independently seeded
layers (--layers, default 16, 10.7 GB) so that a step's weights come from HBM and not from the
256 MB Infinity Cache.  Inputs are resident in HBM before the timed region starts.

Prints one JSON line: whole-job tokens/s, the roofline of the dominant kernel (routed gate/up GEMV,
algorithmic bytes / measured launch duration against the 8 TB/s HBM peak) and the CPU oracle timed
on this host's cores."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
EXPERT_MATRIX_BYTES = 512 * 2048 // 256 * 210   # one Q6_K [512 x 2048] matrix: 860160 B
SHARED_BYTES = 3 * (512 * 2048 // 32 * 34)      # shared expert, Q8_0
ROUTER_BYTES = 256 * 2048 // 32 * 34            # router, Q8_0


MIN_TIMED_STEPS = 320   # the headline's timed region never covers fewer block passes than this (~11 ms)


def routing_margin(logits):
    """min over tokens of p(8th selected) - p(9th): how close the top-8 / top-9 decision of `route_token`
    (crates/xabe-kernels/src/moe/router.rs:32-76) comes to a tie on these logits; float64 softmax on the host."""
    import numpy as np

    l = np.asarray(logits, np.float64)
    e = np.exp(l - l.max(axis=1, keepdims=True))
    p = np.sort(e / e.sum(axis=1, keepdims=True), axis=1)[:, ::-1]
    ls = np.sort(l, axis=1)[:, ::-1]
    return float((p[:, 7] - p[:, 8]).min()), float((ls[:, 7] - ls[:, 8]).min())


def source_digest():
    """Digest of the kernel sources the counter-derived `traffic` figure was taken on: a figure from another
    version of the kernels is reported as stale, not as measured."""
    import hashlib

    h = hashlib.sha256()
    for name in ("decode_block.hip", "decode_kernels.h", "device_common.h", "route_device.h"):
        with open(os.path.join(ROOT, "llmxabe_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def prefill_leg(X, layers, T, reps, bias=None):
    """One prefill configuration of the block (eager launches, HIP events on the launch stream, layers rotated)."""
    import numpy as np
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    blk = X.MoeBlock(g)
    blk.publish_tokens(T)
    x = X.synth_normal_f32(99, T * 2048, 1.0).view(T, 2048)
    ffn_out, l_out = torch.zeros_like(x), torch.zeros_like(x)
    extra = {"logit_bias": bias} if bias is not None else {}
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    L = len(layers)
    with torch.cuda.stream(stream):
        for i in range(2 * L):
            blk.forward(layers[i % L], x, T, ffn_out, l_out, **extra)
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            for i in range(L):
                blk.forward(layers[i], x, T, ffn_out, l_out, **extra)
        e1.record(stream)
        e1.synchronize()
    ms = e0.elapsed_time(e1) / (reps * L)
    ids = blk.buffers().topk_ids().cpu().numpy().reshape(T, 8)
    distinct = len(np.unique(ids))
    byts = distinct * 3 * EXPERT_MATRIX_BYTES + SHARED_BYTES + ROUTER_BYTES + 16384 + T * 2048 * 4 * 3
    flops = T * 57671680
    gbps, tflops = byts / (ms * 1e-3) / 1e9, flops / (ms * 1e-3) / 1e12
    margin_p, margin_l = routing_margin(blk.router_logits().view(T, 256).cpu().numpy())
    counts = np.bincount(ids.ravel(), minlength=256)
    out = {"tokens": T, "block_size": g.block_size, "ms_per_block": ms, "tokens_per_s": T / (ms * 1e-3), "steps": reps * L,
           "layers_rotated": L, "tflops": tflops, "frac_of_mfma_peak": tflops / MFMA_PEAK_TFLOPS, "gbps": gbps,
           "frac_of_hbm_peak": gbps / HBM_PEAK_GBPS, "bound": "mfma" if T >= 4096 else "hbm",
           "distinct_experts": distinct, "algorithmic_bytes_per_block": byts, "flops_per_block": flops,
           "expert_load": {"max": int(counts.max()), "experts_with_at_most_2_tokens": int((counts <= 2).sum())},
           "routing_margin_min": margin_p, "routing_logit_gap_min": margin_l,
           "dtype": "f16 operands, f32 accumulate (router f32)", "launch": "eager",
           "router_bias": "zipf s=1.1 (b_e = -1.1 ln rank_e), seed 5" if bias is not None else None}
    del blk, x, ffn_out, l_out
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--layers", type=int, default=16, help="independent weight sets rotated through")
    ap.add_argument("--tokens", type=int, default=3)
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a hipGraph")
    ap.add_argument("--calibration-copies", type=int, default=0,
                    help="before the timed region, copy a 256 MiB device buffer this many times: a kernel of known "
                         "traffic against which hardware byte counters of the same run are scaled")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the two prefill legs of the headline run")
    ap.add_argument("--no-calibration", action="store_true", help="skip the read / matrix-instruction calibration legs")
    ap.add_argument("--mfma-form", type=int, default=0, choices=[0, 1, 2],
                    help="--workload prefill_*: which grouped-GEMM kernel the routed launches take (2: the "
                         "specialised-wavefront form, same bits, kept for comparison)")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the compact legs of BASELINE's other configurations (decode batch 32, the dense sibling, the 40-layer stack)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--workload", default="decode_b3", choices=["decode_b3"] + sorted(OTHER_WORKLOADS),
                    help="decode_b3 is the headline: the batch-3 decode block (value, roofline), followed by the "
                         "8192-token and the skewed 512-token prefill blocks (the `prefill` object); the others are "
                         "BASELINE's remaining configurations one at a time, for profiles and comparison")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2
    if args.workload != "decode_b3":
        return other_workload(args)

    import numpy as np
    import torch

    import llmxabe_amd as X

    torch.cuda.set_device(0)
    T = args.tokens
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    L = args.layers

    layers = []
    for l in range(L):
        layers.append(make_layer_device_only(X, g, seed=10_000 + 100 * l))
    x = X.synth_normal_f32(99, T * 2048, 1.0).view(T, 2048)   # fp32 N(0,1) activations, resident in HBM
    blk = X.MoeBlock(g)
    blk.publish_tokens(T)
    ffn_out = torch.zeros_like(x)
    l_out = torch.zeros_like(x)
    if args.calibration_copies:
        src = torch.zeros(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(args.calibration_copies):
            dst.copy_(src)
        del src, dst
    torch.cuda.synchronize()   # the generators ran on the default stream; the timed work uses its own

    def one_pass(i):
        blk.forward(layers[i % L], x, T, ffn_out, l_out)

    # ---- timed region: W warmup steps, then K steps (never fewer than MIN_TIMED_STEPS: at 30 us a step, the 20
    # steps a short run asks for are two graph replays, one scheduler hiccup away from noise); whole replays of the
    # L-pass graph, so both counts are rounded up to multiples of L.  HIP events on the launch stream give the
    # figure; the host clock around the same region is reported beside it ----
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(L):
            one_pass(i)
        stream.synchronize()
        graph = None
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(L):
                    one_pass(i)
        reps_w = max(1, (args.warmup + L - 1) // L)
        reps = max(1, (max(args.steps, MIN_TIMED_STEPS) + L - 1) // L)
        steps = reps * L
        for _ in range(reps_w):
            graph.replay() if graph else [one_pass(i) for i in range(L)]
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(reps):
            graph.replay() if graph else [one_pass(i) for i in range(L)]
        e1.record(stream)
        e1.synchronize()
        wall = time.perf_counter() - t0
        dt = e0.elapsed_time(e1) * 1e-3
    ms_per_step = dt / steps * 1e3
    tokens_per_s = T * steps / dt

    # ---- algorithmic bytes of one step (distinct experts from topk_ids of each layer), and how close the routing
    # decision of each pass came to a tie ----
    distinct, margins, gaps = [], [], []
    with torch.cuda.stream(stream):
        for i in range(L):
            one_pass(i)
            stream.synchronize()
            ids = blk.buffers().topk_ids().cpu().numpy().reshape(T, 8)
            distinct.append(len(np.unique(ids)))
            mp, ml = routing_margin(blk.router_logits().view(T, 256).cpu().numpy())
            margins.append(mp)
            gaps.append(ml)
    d_active = float(np.mean(distinct))
    step_bytes = d_active * 3 * EXPERT_MATRIX_BYTES + SHARED_BYTES + ROUTER_BYTES + 16384 + T * 2048 * 4 * 3
    step_gbps = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- the three launches of the block, each timed alone (HIP events on the launch stream, graph replay
    # over the same rotated layers); the dominant one is launch 1: route + routed gate/up, which streams
    # two of the three matrices of every distinct expert selected (and the shared expert's gate/up pair) ----
    chunks = (T + 1) // 2  # token chunks of two share one pass over the router and shared gate/up
    stage_bytes = decode_stage_bytes(T, d_active, chunks)
    stage_us = []
    with torch.cuda.stream(stream):
        one_pass(0)  # leaves layer 0's logits, normalised rows and shared activations for stages 1 and 2
        stream.synchronize()
        for st in range(3):
            def run_stage(i, st=st):
                blk.forward_stage(layers[i % L], x, ffn_out, l_out, st)
            for i in range(L):
                run_stage(i)
            stream.synchronize()
            kgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(kgraph, stream=stream):
                for i in range(L):
                    run_stage(i)
            kgraph.replay()
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            kreps = 20
            e0.record(stream)
            for _ in range(kreps):
                kgraph.replay()
            e1.record(stream)
            e1.synchronize()
            stage_us.append(e0.elapsed_time(e1) * 1e3 / (kreps * L))
    kern_bytes, kern_us = stage_bytes[1], stage_us[1]
    achieved = kern_bytes / (kern_us * 1e-6) / 1e9
    # HBM bytes per launch of the dominant kernel from hardware counters: taken in separate `rocprofv3 --pmc` runs of
    # this command (profiles/moe_block_decode_b3_hbm_traffic.md), valid only for the kernel sources it was taken on
    traffic, traffic_note = None, "no counter profile for this workload"
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath) and T == 3:
        try:
            tj = json.load(open(tpath))
            if tj.get("kernel_source_digest") == source_digest():
                traffic = tj.get("k_decode_up_b3_bytes_per_launch")
                traffic_note = "rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE per dispatch, scaled by a 256 MiB copy (profiles/moe_block_decode_b3_hbm_traffic.md)"
            else:
                traffic_note = "stale: profiles/traffic.json was taken on other kernel sources (digest %s, now %s)" % (
                    tj.get("kernel_source_digest"), source_digest())
        except Exception as e:  # noqa: BLE001
            traffic_note = f"unreadable profiles/traffic.json: {e}"
    stage_names = DECODE_STAGE_NAMES

    out = {
        "metric": "MoE-block tokens/s at 1 GPU; decode HBM GB/s %peak; prefill MFMA util %",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": reps_w * L,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "moe_block_decode_b3" if T == 3 else f"moe_block_decode_b{T}", "tokens": T,
                   "num_experts": 256, "top_k": 8, "hidden": 2048, "intermediate": 512, "expert_quant": "Q6_K",
                   "shared_and_router_quant": "Q8_0", "layers_rotated": L, "launch": "eager" if args.no_graph else "hipGraph"},
        "timing": {"steps_requested": args.steps, "warmup_requested": args.warmup, "steps_timed": steps,
                   "warmup_run": reps_w * L, "min_timed_steps": MIN_TIMED_STEPS,
                   "method": f"HIP events on the launch stream around {reps} replays of a {L}-pass hipGraph "
                             f"(whole replays: both counts are rounded up to multiples of {L}; the timed region is never "
                             f"shorter than {MIN_TIMED_STEPS} steps)",
                   "timed_region_ms": dt * 1e3, "host_clock_ms_per_step": wall / steps * 1e3},
        "decode": {"distinct_experts_per_step": d_active, "algorithmic_bytes_per_step": step_bytes,
                   "block_gbps": step_gbps, "block_frac_of_hbm_peak": step_gbps / HBM_PEAK_GBPS,
                   "roofline_tokens_per_s": T / (step_bytes / (HBM_PEAK_GBPS * 1e9)),
                   "frac_of_roofline": tokens_per_s / (T / (step_bytes / (HBM_PEAK_GBPS * 1e9))),
                   "routing_margin_min": float(np.min(margins)), "routing_logit_gap_min": float(np.min(gaps))},
        "roofline": {"kernel": DECODE_DOMINANT_KERNEL, "bound": "hbm", "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic,
                     "traffic_source": traffic_note,
                     "algorithmic_bytes_per_launch": kern_bytes, "launch_us": kern_us},
        "launches": [{"kernel": n, "launch_us": u, "algorithmic_bytes": int(bts), "gbps": bts / (u * 1e-6) / 1e9}
                     for n, u, bts in zip(stage_names, stage_us, stage_bytes)],
    }
    del graph, blk

    # ---- the prefill half of the metric: the 8192-token chunk (MFMA-bound) and configs[2]'s 512-token chunk under a
    # seeded Zipf(1.1) router bias (HBM-bound), on the first layers of the same weight sets ----
    if not args.no_prefill:
        zipf = torch.from_numpy(X.zipf_logit_bias(256)).cuda()
        out["prefill"] = {"tokens_8192": prefill_leg(X, layers[:2], 8192, 20),
                          "tokens_512_zipf": prefill_leg(X, layers[:4], 512, 40, bias=zipf)}
        out["prefill"]["mfma_util_pct"] = 100.0 * out["prefill"]["tokens_8192"]["frac_of_mfma_peak"]

    if not args.no_calibration:
        out["calibration"] = calibration(X, stream)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(layers[0], g, x, T, args.cpu_seconds)
    # ---- BASELINE's remaining configurations, one compact leg each (the same code `--workload NAME` runs alone):
    # configs[3] decode batch 32 as a block and through the 40-layer stack, configs[4] the dense sibling ----
    if not args.no_configs:
        del layers, x, ffn_out, l_out
        torch.cuda.empty_cache()
        legs = {}
        for name in ("decode_b32", "dense_b1", "dense_b8", "dense_2048", "stack40_b32"):
            r = run_other(args, name)
            leg = {"tokens": r["config"]["tokens"], "ms_per_step": r["ms_per_step"], "tokens_per_s": r["value"], "steps": r["steps"],
                   "algorithmic_bytes_per_step": r["algorithmic_bytes_per_step"], "flops_per_step": r["flops_per_step"],
                   "bound": r["roofline"]["bound"], "achieved": r["roofline"]["achieved"], "unit": r["roofline"]["unit"],
                   "frac": r["roofline"]["frac"]}
            for key in ("layers", "us_per_layer", "layers_rotated", "distinct_experts"):
                if key in r["config"]:
                    leg[key] = r["config"][key]
            if "seam" in r:
                leg["seam"] = r["seam"]
            legs[name] = leg
        out["configs"] = legs
    print(json.dumps(out))
    return 0


DECODE_STAGE_NAMES = ["k_decode_logits (router logits + shared gate/up)", "k_decode_up (route + routed gate/up)",
                      "k_decode_down (routed + shared down, combine)"]
DECODE_DOMINANT_KERNEL = "k_decode_up<Q6_K,hidden 2048> (route + routed gate/up)"


def decode_stage_bytes(T, d_active, chunks):
    """Algorithmic bytes of the three decode launches: every distinct selected expert's matrices once, the router and
    the shared expert's matrices once per launch that reads them (re-reads by further token chunks come out of cache
    and are not algorithmic)."""
    return [ROUTER_BYTES + 2 * (SHARED_BYTES // 3),
            d_active * 2 * EXPERT_MATRIX_BYTES,
            d_active * EXPERT_MATRIX_BYTES + SHARED_BYTES // 3]


def calibration(X, stream):
    """What this box can do, next to the nominal peaks: a pure coalesced 16-byte-per-lane read of 2 GiB (eight times
    the 256 MB Infinity Cache) and a register-resident fp16 matrix-instruction loop, both kernels of this library's
    calibrate.hip; and, for comparison, two library routines."""
    import torch

    with torch.cuda.stream(stream):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        big = torch.ones(1 << 29, dtype=torch.int32, device="cuda")   # 2 GiB
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        X.calibrate_hbm_read(big, sink)
        e0.record(stream)
        for _ in range(5):
            X.calibrate_hbm_read(big, sink)
        e1.record(stream)
        e1.synchronize()
        read_gbps = 5 * big.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9
        half = big[: 1 << 28]
        dst = torch.empty_like(half)
        dst.copy_(half)
        e0.record(stream)
        for _ in range(5):
            dst.copy_(half)
        e1.record(stream)
        e1.synchronize()
        copy_gbps = 5 * 2 * half.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9
        del big, half, dst
        mout = torch.zeros(512 * 1024, dtype=torch.float32, device="cuda")
        X.calibrate_mfma_f16(mout, 2000)
        e0.record(stream)
        mflops = X.calibrate_mfma_f16(mout, 20000)
        e1.record(stream)
        e1.synchronize()
        mfma_tflops = mflops / (e0.elapsed_time(e1) * 1e-3) / 1e12
        ma = torch.randn(8192, 8192, device="cuda", dtype=torch.float16)
        mb = torch.randn(8192, 8192, device="cuda", dtype=torch.float16)
        torch.matmul(ma, mb)
        e0.record(stream)
        for _ in range(5):
            torch.matmul(ma, mb)
        e1.record(stream)
        e1.synchronize()
        gemm_tflops = 5 * 2 * 8192 ** 3 / (e0.elapsed_time(e1) * 1e-3) / 1e12
        del ma, mb
    return {"hbm_read_gbps": read_gbps, "hbm_read_what": "coalesced 16-byte-per-lane read of 2 GiB (xabe_calibrate_hbm_read)",
            "mfma_f16_tflops": mfma_tflops, "mfma_f16_what": "register-resident v_mfma_f32_32x32x16_f16 loop, two wavefronts per SIMD (xabe_calibrate_mfma_f16)",
            "device_copy_gbps": copy_gbps, "device_copy_what": "torch copy of 1 GiB, bytes read + written",
            "fp16_gemm_tflops": gemm_tflops, "fp16_gemm_what": "torch.matmul 8192^3 fp16 (hipBLASLt)"}


MFMA_PEAK_TFLOPS = 2500.0
# name -> (kind, tokens, layers rotated): the MoE block at other widths and the dense sibling
OTHER_WORKLOADS = {"decode_b32": ("moe", 32, 16), "prefill_512": ("moe", 512, 4), "prefill_512_uniform": ("moe", 512, 4),
                   "prefill_8192": ("moe", 8192, 2),
                   # the 40-layer stack (26.4 GB of experts resident), each block's l_out the next block's input
                   "stack40_b3": ("stack", 3, 40), "stack40_b32": ("stack", 32, 40), "stack40_8192": ("stack", 8192, 40),
                   "dense_b1": ("dense", 1, 4), "dense_b8": ("dense", 8, 4), "dense_2048": ("dense", 2048, 2),
                   # the LM head (2048 -> 248 320, Q8_0: 540 MB per pass), two copies rotated
                   "lm_head_b1": ("lm_head", 1, 2), "lm_head_b3": ("lm_head", 3, 2), "lm_head_b8": ("lm_head", 8, 2)}


def other_workload(args) -> int:
    print(json.dumps(run_other(args, args.workload)))
    return 0


def run_other(args, workload) -> dict:
    """One of BASELINE's other configurations: the whole block, eager launches, HIP events on the launch
    stream over rotated layers.  One JSON line in the headline's format; the roofline is the block's own
    (algorithmic bytes or flops of a pass over its duration), not one kernel's."""
    import numpy as np
    import torch

    import llmxabe_amd as X

    torch.cuda.set_device(0)
    kind, T, L = OTHER_WORKLOADS[workload]
    if kind == "lm_head":
        return lm_head_workload(args, T, L)
    if kind == "stack":
        return stack_workload(args, workload, T, L)
    if kind == "moe":
        g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
        layers = [make_layer_device_only(X, g, seed=10_000 + 100 * l) for l in range(L)]
        blk = X.MoeBlock(g)
        blk.set_mfma_form(getattr(args, "mfma_form", 0))
        blk.publish_tokens(T)
        width = 2048
    else:
        H, I = 5120, 17408
        q = X.ExpertQuant.Q6K
        layers = []
        for l in range(L):
            t = [X.QuantTensor(X.synth_quant(q, 41 + 10 * l + j, H * I, 0.02), q) for j in range(3)]
            layers.append(X.DenseFfnLayerWeights(1.0 + X.synth_normal_f32(44 + 10 * l, H, 0.1), t[0], t[1], t[2]))
        blk = X.DenseFfnBlock(H, I, T)
        width = H
    x = X.synth_normal_f32(99, T * width, 1.0).view(T, width)
    ffn_out, l_out = torch.zeros_like(x), torch.zeros_like(x)
    if args.calibration_copies:   # a kernel of known traffic for counter runs (see the headline's option)
        src = torch.zeros(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(args.calibration_copies):
            dst.copy_(src)
        del src, dst
    extra = {}
    if workload == "prefill_512":
        # the skewed configuration: a seeded Zipf(s = 1.1) bias over the experts, added to the router logits before
        # routing (b_e = -s ln(rank_e) over a seeded permutation of the experts, i.e. selection odds proportional to rank^-1.1)
        extra["logit_bias"] = torch.from_numpy(X.zipf_logit_bias(256)).cuda()
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    reps_w = max(1, min(args.warmup, 64) // L)
    reps = max(1, min(max(args.steps, 64), 64 if T >= 512 else 320) // L)   # (never fewer than 64 block passes)
    with torch.cuda.stream(stream):
        for _ in range(reps_w):
            for i in range(L):
                blk.forward(layers[i], x, T, ffn_out, l_out, **extra)
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            for i in range(L):
                blk.forward(layers[i], x, T, ffn_out, l_out, **extra)
        e1.record(stream)
        e1.synchronize()
    steps = reps * L
    ms = e0.elapsed_time(e1) / steps
    if kind == "moe":
        ids = blk.buffers().topk_ids().cpu().numpy().reshape(T, 8)
        distinct = len(np.unique(ids))
        byts = distinct * 3 * EXPERT_MATRIX_BYTES + SHARED_BYTES + ROUTER_BYTES + 16384 + T * 2048 * 4 * 3
        flops = T * 57671680
        cfg = {"workload": "moe_block_" + workload, "tokens": T, "num_experts": 256, "top_k": 8, "hidden": 2048,
               "intermediate": 512, "expert_quant": "Q6_K", "shared_and_router_quant": "Q8_0", "layers_rotated": L,
               "launch": "eager", "distinct_experts": distinct,
               "router_bias": "zipf s=1.1 (b_e = -1.1 ln rank_e), seed 5" if extra else None}
        if extra:
            counts = np.bincount(ids.ravel(), minlength=256)
            cfg["expert_load"] = {"max": int(counts.max()), "experts_with_at_most_2_tokens": int((counts <= 2).sum())}
    else:
        byts = 3 * 5120 * 17408 // 256 * 210
        flops = T * 3 * 2 * 5120 * 17408
        cfg = {"workload": "dense_ffn_" + workload, "tokens": T, "hidden": 5120, "intermediate": 17408,
               "quant": "Q6_K", "layers_rotated": L, "launch": "eager"}
    gbps, tflops = byts / (ms * 1e-3) / 1e9, flops / (ms * 1e-3) / 1e12
    mfma_bound = workload in ("prefill_8192", "dense_2048")
    roof = ({"kernel": "whole block", "bound": "mfma", "achieved": tflops, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
             "frac": tflops / MFMA_PEAK_TFLOPS, "traffic": None} if mfma_bound else
            {"kernel": "whole block", "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": gbps / HBM_PEAK_GBPS, "traffic": None})
    del blk, layers, x, ffn_out, l_out
    torch.cuda.empty_cache()
    return {
        "metric": "MoE-block tokens/s at 1 GPU; decode HBM GB/s %peak; prefill MFMA util %", "value": T / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": reps_w * L, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 operands, f32 accumulate" if T >= 64 else "f32",
        "data": "synthetic", "config": cfg, "roofline": roof, "algorithmic_bytes_per_step": byts, "flops_per_step": flops,
        "cpu_baseline": None}


def stack_workload(args, workload, T, L) -> dict:
    """L independently seeded MoE layers resident at once, one pass of T tokens through all of them per step:
    layer l's l_out (residual + block output) is layer l + 1's input, with the RMSNorm between them either as the
    next block's first step (`value`: the reference-shaped calls) or folded into the launch that finishes l_out (the
    `seam` object: xabe_moe_block_forward_seam, same bits).  Ping-pong activation buffers, HIP events on the launch
    stream; at decode widths the whole pass is one hipGraph (as a decode engine would replay it: eager launches of
    three ~10 us kernels per layer are bound by the host), wider passes are launched eagerly."""
    import numpy as np
    import torch

    import llmxabe_amd as X

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    layers = [make_layer_device_only(X, g, seed=20_000 + 100 * l) for l in range(L)]
    blk = X.MoeBlock(g)
    blk.publish_tokens(T)
    x0 = X.synth_normal_f32(99, T * 2048, 1.0).view(T, 2048)
    bufs = [torch.zeros_like(x0), torch.zeros_like(x0)]
    ffn_out = torch.zeros_like(x0)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()

    def one_pass(seam=False):
        cur = x0
        for i, w in enumerate(layers):
            nxt = bufs[i & 1]
            if seam:  # one handle serves every layer: the tail writes the block's own normalised rows
                blk.forward_seam(w, cur, T, None, nxt, input_normed=i > 0, skip_readback=True,
                                 next_norm_weight=layers[i + 1].post_norm if i + 1 < L else None)
            else:
                blk.forward(w, cur, T, ffn_out, nxt)
            cur = nxt
        return cur

    reps_w, reps = max(1, min(args.warmup, 4)), max(2, min(args.steps, 16 if T < 512 else 4))
    use_graph = T <= 32 and not args.no_graph
    times, outs = {}, {}
    with torch.cuda.stream(stream):
        for seam in (False, True):
            for _ in range(reps_w):
                out = one_pass(seam)
            stream.synchronize()
            run = lambda: one_pass(seam)  # noqa: E731
            if use_graph:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    one_pass(seam)
                graph.replay()
                stream.synchronize()
                run = graph.replay
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(reps):
                run()
            e1.record(stream)
            e1.synchronize()
            times[seam] = e0.elapsed_time(e1) / reps
            outs[seam] = out.clone()
    ms = times[False]
    finite = bool(torch.isfinite(outs[False]).all().item())
    same_bits = bool(torch.equal(outs[False].view(torch.int32), outs[True].view(torch.int32)))
    flops = L * T * 57671680
    weight_bytes = L * (256 * 3 * EXPERT_MATRIX_BYTES + SHARED_BYTES + ROUTER_BYTES)
    tflops = flops / (ms * 1e-3) / 1e12
    mfma = T >= 64
    # algorithmic bytes of a pass: every layer's distinct selected experts (read back layer by layer, untimed)
    byts, cur = 0, x0
    for i, w in enumerate(layers):
        blk.forward(w, cur, T, ffn_out, bufs[i & 1])
        cur = bufs[i & 1]
        distinct = len(np.unique(blk.buffers().topk_ids().cpu().numpy().reshape(T, 8)))
        byts += distinct * 3 * EXPERT_MATRIX_BYTES + SHARED_BYTES + ROUTER_BYTES + 16384 + T * 2048 * 4 * 3
    gbps = byts / (ms * 1e-3) / 1e9
    roof = ({"kernel": "whole stack", "bound": "mfma", "achieved": tflops, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
             "frac": tflops / MFMA_PEAK_TFLOPS, "traffic": None} if mfma else
            {"kernel": "whole stack", "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": gbps / HBM_PEAK_GBPS, "traffic": None})
    seam_ms = times[True]
    del blk, layers, bufs, ffn_out, outs
    torch.cuda.empty_cache()
    return {
        "metric": "MoE-block tokens/s at 1 GPU; decode HBM GB/s %peak; prefill MFMA util %", "value": T / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": reps, "warmup": reps_w, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 operands, f32 accumulate" if mfma else "f32", "data": "synthetic",
        "config": {"workload": "moe_stack_" + workload, "layers": L, "tokens": T, "num_experts": 256, "top_k": 8,
                   "hidden": 2048, "intermediate": 512, "expert_quant": "Q6_K", "shared_and_router_quant": "Q8_0",
                   "resident_weight_bytes": weight_bytes, "launch": "hipGraph" if use_graph else "eager", "us_per_layer": ms * 1e3 / L,
                   "output_finite": finite},
        "seam": {"what": "the same pass with every layer boundary's RMSNorm folded into the launch that finishes l_out "
                         "(xabe_moe_block_forward_seam; no ffn_out / routed read-back tensors)",
                 "ms_per_step": seam_ms, "us_per_layer": seam_ms * 1e3 / L, "tokens_per_s": T / (seam_ms * 1e-3),
                 "speedup": ms / seam_ms, "same_bits_as_unfused": same_bits},
        "roofline": roof, "algorithmic_bytes_per_step": byts, "flops_per_step": flops, "cpu_baseline": None}


def lm_head_workload(args, T, L) -> dict:
    """The LM-head GEMV over the real head's shape (Q8_0), logits for T tokens per step; HIP events on the
    launch stream; the CPU leg is the oracle's sequential gemv over a slice of the vocabulary."""
    import time

    import numpy as np
    import torch

    import llmxabe_amd as X

    torch.cuda.set_device(0)
    g = X.LmHeadGeometry.qwen3_6(T)
    heads = [X.HeadTensor.q8_0(X.synth_quant(X.ExpertQuant.Q8_0, 500 + l, g.elements(), 0.02)) for l in range(L)]
    k = X.LmHeadKernels(g)
    x = X.synth_normal_f32(99, T * g.hidden, 1.0).view(T, g.hidden)
    logits = torch.zeros(T, g.vocab, device="cuda")
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    reps_w, reps = max(1, min(args.warmup, 32) // L), max(1, min(args.steps, 128) // L)
    with torch.cuda.stream(stream):
        for _ in range(reps_w):
            for i in range(L):
                k.forward(heads[i], x, T, logits)
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            for i in range(L):
                k.forward(heads[i], x, T, logits)
        e1.record(stream)
        e1.synchronize()
    steps = reps * L
    ms = e0.elapsed_time(e1) / steps
    byts = g.weight_bytes_read(T) + T * g.hidden * 4 + T * g.vocab * 4
    gbps = byts / (ms * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        import oracle

        rows = 16384
        raw = heads[0].bytes[:rows * g.row_bytes()].cpu().numpy()
        w = oracle.dequantize_row(1, raw)
        xs = x.cpu().numpy()
        t0, n = time.perf_counter(), 0
        while time.perf_counter() - t0 < min(args.cpu_seconds, 10.0):
            oracle.gemv(w, rows, g.hidden, xs[n % T])
            n += 1
        dt = time.perf_counter() - t0
        cpu = {"value": n * rows / g.vocab / dt, "unit": "tokens/s", "cores": 1, "kind": "port",
               "sample": f"sequential gemv over {rows} of the 248320 rows (dequantised beforehand), {n} token passes, scaled to the whole vocabulary"}
    return ({
        "metric": "LM-head tokens/s at 1 GPU; HBM GB/s %peak", "value": T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
        "steps": steps, "warmup": reps_w * L, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "lm_head_b%d" % T, "tokens": T, "hidden": g.hidden, "vocab": g.vocab, "format": "Q8_0",
                   "weight_passes": g.weight_passes(T), "heads_rotated": L, "launch": "eager"},
        "roofline": {"kernel": "k_lm_head_quant", "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": gbps / HBM_PEAK_GBPS, "traffic": None},
        "algorithmic_bytes_per_step": byts, "cpu_baseline": cpu})


def make_layer_device_only(X, g, seed):
    """Seeded device tensors of one layer (same definition as tests/util.make_layer, no host copy)."""
    ROLE = dict(post_norm=1, router=2, gate=3, up=4, down=5, shared_gate_inp=6, sgate=7, sup=8, sdown=9)
    E, H, I = g.num_experts, g.hidden, g.intermediate
    n = E * I * H
    q6, q8 = X.ExpertQuant.Q6K, X.ExpertQuant.Q8_0
    qt = lambda q, role, count: X.QuantTensor(X.synth_quant(q, seed + ROLE[role], count, 0.02), q)
    return X.MoeLayerWeights(
        1.0 + X.synth_normal_f32(seed + ROLE["post_norm"], H, 0.1),
        X.synth_quant(q8, seed + ROLE["router"], E * H, 0.02), q8,
        qt(q6, "gate", n), qt(q6, "up", n), qt(q6, "down", n),
        X.synth_normal_f32(seed + ROLE["shared_gate_inp"], H, 0.02),
        qt(q8, "sgate", I * H), qt(q8, "sup", I * H), qt(q8, "sdown", I * H))


def cpu_baseline(w, g, x, T, budget_s):
    """The CPU oracle (a C port of the reference's scalar path) on this host: the same block, same
    layer-0 weights, same T tokens, repeated until about `budget_s` seconds of CPU work are spent."""
    import oracle

    c = lambda t: t.cpu().numpy()
    host = oracle.MoeWeights(
        num_experts=g.num_experts, top_k=g.experts_per_token, hidden=g.hidden, intermediate=g.intermediate, eps=1e-6,
        post_norm=c(w.post_norm), router_f32=None, router_q8=c(w.router), gate_exps=c(w.gate_exps.bytes),
        up_exps=c(w.up_exps.bytes), down_exps=c(w.down_exps.bytes), shared_gate_inp=c(w.shared_gate_inp),
        shared_gate=c(w.shared_gate.bytes), shared_up=c(w.shared_up.bytes), shared_down=c(w.shared_down.bytes))
    xs = c(x)[:T]

    def run(threads, budget):
        n, t0, deq, mv = 0, time.perf_counter(), 0.0, 0.0
        while True:
            r = oracle.moe_block_forward(host, xs, threads=threads)
            n += 1
            deq += r.seconds_dequant
            mv += r.seconds_matvec
            el = time.perf_counter() - t0
            if el >= budget or n >= 200:
                return n, el, deq, mv

    n1, el1, deq1, mv1 = run(1, budget_s * 0.7)
    cores = min(oracle.num_threads(), 16)   # the box's CPU share for one GPU is 16 cores, whatever nproc shows
    nt, elt, _, _ = run(cores, budget_s * 0.3)
    return {"value": T * n1 / el1, "unit": "tokens/s", "cores": 1, "kind": "port", "host_nproc": os.cpu_count(),
            "sample": f"{n1} passes of the same {T}-token block on layer 0 (dequantise selected experts + sequential "
                      f"fp32 matvecs), {el1:.1f} s; dequant {deq1 / n1 * 1e3:.0f} ms + matvec {mv1 / n1 * 1e3:.0f} ms per pass",
            "openmp": {"value": T * nt / elt, "cores": cores, "passes": nt, "seconds": elt}}


if __name__ == "__main__":
    sys.exit(main())
