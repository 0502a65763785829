#!/usr/bin/env python3
"""Tree-attention decode benchmark on one MI355X.

One "step" is one ``fasttree_decode`` call (stage 1 for both phases + stage 2) over the
3-level tree N=[1,10,400], C=[4000,400,40], 32 query / 8 KV heads, head_dim 128, fp16,
400 decode requests, paged KV pool with shuffled slots (the configuration the headline
target is quoted on).  The planner runs once, outside the timed region, as in the
reference bench (kernel_bench/benchmark.py:88-127).

Prints ONE JSON line on stdout:
  value        median latency of one decode call in microseconds, measured with events
               on the launch stream, every call preceded by a cache flush as the reference's
               timer does it (triton.testing.do_bench, kernel_bench/benchmark.py:35,59): a
               flush buffer is rewritten, here 1 GiB instead of 256 MB because this part has
               256 MB of Infinity Cache; 200 such calls whatever --steps is.  `value_method`
               in the line names the method ("cold_median_after_write_flush") and does not
               change between builds.  The call after such a flush also pays for writing the
               buffer's dirty lines back (up to 288 MB on this part) as its own reads evict
               them; the same call after a flush that rewrites the buffer AND reads it back
               (clean lines in the caches, the pool still not in them) is reported beside it
               as latency_us.cold_clean_median.
  ms_per_step  wall clock of exactly --steps back-to-back calls / steps (warm caches,
               launch overhead included), after --warmup untimed calls.  Before those the
               device is kept busy with the same call for 200 ms (`device_warmup_ms` in the
               line): its clocks settle only after about 100 ms of work, and --warmup counts
               calls, not time (do_bench warms up by time, too).
  roofline     the dominant kernel of the call; its duration is the mean over the timed steps
               of the event-to-event time around its launch.
  cpu_baseline the reference's no-sharing formulation (per-request gathered KV, PyTorch
               ops) on this box's host cores, on a bounded sample of requests.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for extra in ("fasttree-artifact_amd", "oracle", os.path.join("tests", "golden")):
    sys.path.insert(0, os.path.join(ROOT, extra))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
DEVICE_WARMUP_MS = 200.0       # untimed calls before the --warmup steps, until the device's clocks have settled
COLD_CALLS = 200               # flush + call repetitions behind `value` (their median)
# How `value` is taken; fixed, so that the figure compares across builds: the median over COLD_CALLS
# calls, each after the flush buffer has been rewritten (and not read back), as do_bench does it.
VALUE_METHOD = "cold_median_after_write_flush"
MFMA_PEAK_TFLOPS = 2500.0      # dense fp16 / bf16

WORKLOADS = {
    # name: (nodes per level, context per level, Hq, Hkv, dtype)
    "c1": ([1, 16], [1024, 128], 32, 32, "fp16"),
    "c2": ([1, 64], [4096, 256], 32, 8, "fp16"),
    "c3": ([1, 10, 400], [4000, 400, 40], 32, 8, "fp16"),
    "c4": ([1, 2048], [512, 1024], 32, 8, "bf16"),
    # seeded irregular tree (5 levels, fan-out U[1,8], lengths log-uniform [16,2048], <= 1024 leaves); sizes = seed
    "c5": (0, None, 64, 8, "fp16"),
}

# Planner arguments.  "reference" = the values the reference bench passes
# (kernel_bench/benchmark.py:246-254, run_benchmark.sh:46-53: query tiles (64 // g, 16 // g)).
# "mi355x" = the same tiles with the parallelism thresholds sized for 256 compute units instead of
# an H100's 132 and a KV split of 256 instead of 128 tokens for phases short of parallelism (half
# the partial rows per request; the launches that take it are small and bound by their
# partials); "wide" = as "mi355x" with a first-phase query tile of 256 // g requests (kept for
# comparison: slower than "mi355x" over the reference's sweep now that query tiles are joined).
# HBM bytes per launch of the dominant kernel (read + write) measured with rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE, each scaled by what the same counter reads for a plain copy of known size;
# the figure is read from the tracked summary of those runs, profiles/<kernel>_<workload>_<dtype>.txt,
# where a line "hbm traffic per launch [<preset>]: <bytes> bytes" records it (None without that line).
def measured_traffic(workload, preset, kernel, dtype):
    import re
    path = os.path.join(ROOT, "profiles", f"{kernel}_{workload}_{dtype}.txt")
    if not os.path.exists(path):
        return None
    for line in open(path):
        m = re.match(r"hbm traffic per launch \[(\w+)\]:\s*([0-9.eE+]+) bytes", line.strip())
        if m and m.group(1) == preset:
            return float(m.group(2))
    return None


PRESETS = {
    "reference": dict(q_tiles=None, kv_tiles=(32, 32), kv_splits=(1024, 128), thr1=(132, 528), thr2=(132, 132),
                      launch_order=False),
    "mi355x": dict(q_tiles=None, kv_tiles=(32, 32), kv_splits=(1024, 256), thr1=(256, 1024), thr2=(256, 256),
                   launch_order=True),
    "wide": dict(q_tiles="wide", kv_tiles=(32, 32), kv_splits=(1024, 256), thr1=(256, 1024), thr2=(256, 256),
                 launch_order=True),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_problem(name, preset, device, seed=0):
    import torch
    from cases import build_tree
    from fasttree_hip import planner
    from fasttree_hip.inputs import make_decode_inputs
    from fasttree_hip.planner import FastTreeParams, fasttree_preparation

    sizes, lens, hq, hkv, dt = WORKLOADS[name]
    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16}[dt]
    spec = {"kind": "irregular", "seed": sizes} if lens is None else {"kind": "regular", "sizes": sizes, "lens": lens}
    tree, ptrs, batch = build_tree(spec)
    big = ptrs[-1] * hkv * 128 > (1 << 28)
    inp = make_decode_inputs(tree, hq, hkv, 128, device=device, dtype=dtype, seed=seed, shuffle_slots=True,
                             host_rng=not big)
    g = hq // hkv
    cfg = PRESETS[preset]
    if cfg["q_tiles"] == "wide":
        q_tiles = [max(1, 256 // g), max(1, 16 // g)]
    elif cfg["q_tiles"]:
        q_tiles = list(cfg["q_tiles"])
    else:
        q_tiles = [max(1, 64 // g), max(1, 16 // g)]
    params = FastTreeParams()
    params.set_values(0.66, 0.33, 0.1)
    params.set_q_tile_sizes(list(q_tiles))
    params.set_kv_tile_sizes(list(cfg["kv_tiles"]))
    params.set_kv_group_num(g)
    planner.VERBOSE = False
    t0 = time.perf_counter()
    aux, _ = fasttree_preparation(tree, inp.KV_ptrs, batch, hq, hkv, 128, list(cfg["kv_splits"]), list(cfg["thr1"]),
                                  list(cfg["thr2"]), params, device=device, kv_slot_map=inp.slot_map,
                                  launch_order=cfg.get("launch_order", True))
    plan_ms = (time.perf_counter() - t0) * 1e3
    elem = 2
    total = ptrs[-1]
    algo_bytes = total * hkv * 128 * 2 * elem + 2 * batch * hq * 128 * elem
    algo_flops = 4 * hq * 128 * sum(len(t.requests) * t.seqlen for t in tree)
    return dict(tree=tree, inp=inp, aux=aux, q_tiles=q_tiles, kv_tiles=list(cfg["kv_tiles"]), hq=hq, hkv=hkv,
                batch=batch, dtype=dt, algo_bytes=algo_bytes, algo_flops=algo_flops, plan_ms=plan_ms, total=total)


def quantiles(xs):
    xs = sorted(xs)
    pick = lambda f: xs[min(len(xs) - 1, int(f * len(xs)))]
    return statistics.median(xs), pick(0.2), pick(0.8)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c3", choices=list(WORKLOADS))
    ap.add_argument("--preset", default="mi355x", choices=list(PRESETS))
    ap.add_argument("--q-tiles", default=None, help="override the preset's query tile sizes, e.g. 64,4")
    ap.add_argument("--kv-splits", default=None, help="override the preset's KV split sizes, e.g. 1024,128")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gathered", action="store_true")
    ap.add_argument("--phase", default="both", choices=["both", "wide", "narrow"],
                    help="with --profile-only: launch only the first stage, restricted to the block programs "
                         "(wide) or to the vnodes served one wave each (narrow), for per-phase kernel traces")
    ap.add_argument("--profile-only", action="store_true",
                    help="run warm-up + steps back to back and exit (for rocprofv3)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a plain 256 MiB device copy a few times and exit: the known-size kernel the "
                         "FETCH_SIZE / WRITE_SIZE counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU; --gpus above 1 is not supported "
            "(the path shards by KV head without communication; no multi-GPU figure is produced).")
        sys.exit(2)

    import torch
    import fasttree_oracle as oracle
    from fasttree_hip.decode import (fasttree_decode, fasttree_decode_stage1, fasttree_decode_stage2,
                                     gathered_decode)
    from fasttree_hip.inputs import gather_per_request

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.calibrate_copy:
        src = torch.ones(1 << 26, dtype=torch.int32, device=device)   # 256 MiB
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        log("calibrate-copy: 5 copies of 268435456 bytes (read 256 MiB + write 256 MiB each)")
        return
    if args.q_tiles or args.kv_splits:
        custom = dict(PRESETS[args.preset])
        if args.q_tiles:
            custom["q_tiles"] = tuple(int(x) for x in args.q_tiles.split(","))
        if args.kv_splits:
            custom["kv_splits"] = tuple(int(x) for x in args.kv_splits.split(","))
        PRESETS["custom"] = custom
        args.preset = "custom"
    prob = build_problem(args.workload, args.preset, device)
    inp, aux = prob["inp"], prob["aux"]
    scale = 1.0 / math.sqrt(128)
    o = torch.empty_like(inp.Q)

    def step():
        fasttree_decode(inp.Q, inp.K_pool, inp.V_pool, o, *aux, prob["q_tiles"], prob["kv_tiles"], scale)

    nums, offs = aux[11], aux[12]  # (the phase list carries the program table: passed as it is)
    if args.phase != "both":
        if not args.profile_only:
            log("bench.py: --phase is for --profile-only runs")
            sys.exit(2)
        from fasttree_hip.launch_schedule import LaunchPhases
        part = LaunchPhases([nums[0], 0] if args.phase == "wide" else [0, nums[1]])
        part.narrow_table = getattr(nums, "narrow_table", None)
        if args.phase == "wide":
            part.prog_table = getattr(nums, "prog_table", None)
            part.num_programs = getattr(nums, "num_programs", 0)
            part.prog_records = getattr(nums, "prog_records", None)
        elif getattr(nums, "narrow_in_programs", 0):
            log("bench.py: the narrow vnodes of this plan are served inside the block programs")
            sys.exit(2)
        nums = part

    def stage1():
        fasttree_decode_stage1(inp.Q, inp.K_pool, inp.V_pool, *aux[:6], scale, aux[9], aux[10], nums, offs,
                               prob["q_tiles"], prob["kv_tiles"])

    def stage2():
        fasttree_decode_stage2(aux[6], aux[7], aux[8], aux[9], aux[10], o)

    # The timed region: exactly --steps decode calls back to back.  It is run twice: once bare
    # for the wall clock, once more as its two launches (what ft_decode enqueues) with an event on
    # the launch stream before, between and after, for the per-kernel durations -- the events
    # themselves cost a few microseconds per step, which must not leak into ms_per_step.
    if args.phase != "both":
        t_end = time.perf_counter() + DEVICE_WARMUP_MS * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(16):
                stage1()
            torch.cuda.synchronize()
        for _ in range(args.warmup + args.steps):
            stage1()
        torch.cuda.synchronize()
        log(f"profile-only: {args.warmup + args.steps} stage-1 launches of the {args.phase} phase, vnodes {list(nums)}")
        return
    # The device's clocks settle only after about 100 ms of continuous work (measured: 68 us per
    # step in the first 20 ms of a process, 62 us from 100 ms on), and --warmup counts steps, not
    # time: keep the device busy with the same call for DEVICE_WARMUP_MS first, as
    # triton.testing.do_bench warms up by time (kernel_bench/benchmark.py:59), then do the
    # --warmup steps and time exactly --steps.
    t_end = time.perf_counter() + DEVICE_WARMUP_MS * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(16):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    host_us = (time.perf_counter() - t0) * 1e6 / args.steps   # enqueue only: wrapper + ctypes + two launches
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    for m in marks:
        m[0].record(); stage1(); m[1].record(); stage2(); m[2].record()
    torch.cuda.synchronize()
    per_launch = {"stage1": statistics.mean(m[0].elapsed_time(m[1]) for m in marks) * 1e3,
                  "stage2": statistics.mean(m[1].elapsed_time(m[2]) for m in marks) * 1e3}
    if args.profile_only:
        log(f"profile-only: {args.steps} steps, {wall_ms * 1e3:.1f} us/step wall, launches {per_launch}")
        return

    # ---- parity of this very run against the CPU oracle on a request sample
    sample = list(range(0, prob["batch"], max(1, prob["batch"] // 16)))
    want = oracle.dense_attention(inp.Q[sample].cpu(), inp.K_pool.cpu(), inp.V_pool.cpu(),
                                  [inp.path_tokens[r] for r in sample], scale)
    diff = (o[sample].cpu().double() - want).abs().reshape(len(sample), -1)
    parity = {"max_abs": float(diff.max()), "mean_abs": float(diff.mean(dim=1).max()), "requests_checked": len(sample)}
    # (the bar of the parity tests; bf16 outputs are allowed their storage rounding on top, |o| * 2**-8)
    allowed = 2e-3 + (float(want.abs().max()) * 2.0 ** -8 if prob["dtype"] == "bf16" else 0.0)
    parity["passed"] = bool(parity["max_abs"] <= allowed and parity["mean_abs"] <= 1e-3 + (allowed - 2e-3))
    if prob["dtype"] == "bf16":
        # like for like: the reference kernels' arithmetic evaluated in bfloat16 on the same plan (P rounded to
        # bfloat16, fp32 accumulation, bfloat16 output; kernel_bench/fasttree.py:391, 405-413, 534-546), held to
        # the plain bar.  max_abs / mean_abs above are the raw figures against fp64.
        import numpy as np
        paths = [inp.path_tokens[r] for r in sample]
        uniq = np.unique(np.concatenate(paths))
        remap = {int(s): i for i, s in enumerate(uniq)}
        rows = torch.from_numpy(uniq).to(device)
        same = oracle.decode_arith_for_requests(inp.Q[sample].cpu(), inp.K_pool[rows].cpu(), inp.V_pool[rows].cpu(),
                                                [t.cpu().numpy() for t in aux[:9]], sample, 32, scale, remap=remap)
        like = (o[sample].cpu().double() - same.double()).abs().reshape(len(sample), -1)
        parity["like_for_like_bf16"] = {"max_abs": float(like.max()), "mean_abs": float(like.mean(dim=1).max())}
        parity["passed"] = bool(parity["passed"] and like.max() <= 2e-3 and like.mean(dim=1).max() <= 1e-3)

    # ---- cold-cache latency per call (events on the launch stream, flush before every call)
    flush = torch.empty(1 << 28, dtype=torch.int32, device=device)     # 1 GiB

    def flush_caches(clean=True):
        flush.zero_()          # evicts the pool from L2 and the Infinity Cache ...
        if clean:
            flush.sum()        # ... and reading the buffer back leaves clean lines behind
    reps = COLD_CALLS
    cold, warm = [], []
    for _ in range(reps):
        flush_caches(clean=False)        # the reference's method: the flush buffer is rewritten, nothing else
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); step(); e1.record()
        e1.synchronize()
        cold.append(e0.elapsed_time(e1) * 1e3)
    cold_clean = []
    for _ in range(max(30, reps // 4)):
        flush_caches(clean=True)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); step(); e1.record()
        e1.synchronize()
        cold_clean.append(e0.elapsed_time(e1) * 1e3)
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); step(); e1.record()
        e1.synchronize()
        warm.append(e0.elapsed_time(e1) * 1e3)
    cold_med, cold_p20, cold_p80 = quantiles(cold)
    warm_med, _, _ = quantiles(warm)

    dominant = max(per_launch, key=per_launch.get)

    # algorithmic work of the stage-1 launch (both phases run in one kernel): every unique KV
    # element read once, Q read once; stage 2 is scratch traffic only
    elem = 2
    rows = aux[3].numel()
    work = {
        "stage1": dict(bytes=prob["total"] * prob["hkv"] * 128 * 2 * elem + prob["batch"] * prob["hq"] * 128 * elem,
                       flops=prob["algo_flops"]),
        "stage2": dict(bytes=rows * prob["hq"] * (128 + 1) * 4 + prob["batch"] * prob["hq"] * 128 * elem, flops=0),
    }
    dom_us = per_launch[dominant]
    dom = work[dominant]
    traffic = measured_traffic(args.workload, args.preset, dominant, prob["dtype"])
    mfma_frac = dom["flops"] / (dom_us * 1e-6) / 1e12 / MFMA_PEAK_TFLOPS
    hbm_frac = dom["bytes"] / (dom_us * 1e-6) / 1e9 / HBM_PEAK_GBS
    if mfma_frac >= hbm_frac:
        roofline = {"kernel": dominant, "bound": "mfma", "achieved": dom["flops"] / (dom_us * 1e-6) / 1e12,
                    "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": mfma_frac, "traffic": traffic,
                    "avg_launch_us": dom_us}
    else:
        roofline = {"kernel": dominant, "bound": "hbm", "achieved": dom["bytes"] / (dom_us * 1e-6) / 1e9,
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": hbm_frac, "traffic": traffic, "avg_launch_us": dom_us}

    # ---- the no-sharing baseline on the GPU: per-request gathered cache through the same kernels
    gathered = None
    if not args.no_gathered and args.workload != "c4":
        k_cache, v_cache, lens = gather_per_request(inp)
        og = torch.empty_like(inp.Q)
        nsplit = (k_cache.shape[1] + 511) // 512
        mo = torch.empty((prob["batch"] * nsplit, prob["hq"], 128), dtype=torch.float32, device=device)
        ml = torch.empty((prob["batch"] * nsplit, prob["hq"]), dtype=torch.float32, device=device)
        ts = []
        for i in range(13):
            flush_caches(clean=False)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(); gathered_decode(inp.Q, k_cache, v_cache, lens, og, scale, 512, mo, ml); e1.record()
            e1.synchronize()
            if i >= 3:
                ts.append(e0.elapsed_time(e1) * 1e3)
        gbytes = int(lens.sum().item()) * prob["hkv"] * 128 * 2 * elem
        gathered = {"latency_us": statistics.median(ts), "bytes": gbytes,
                    "GBps": gbytes / (statistics.median(ts) * 1e-6) / 1e9,
                    "max_abs_vs_tree": float((og.float() - o.float()).abs().max())}
        del k_cache, v_cache, mo, ml

    # ---- the reference's own no-sharing ablation: same kernels, same pool, a plan in which every
    # leaf absorbs its whole path (alpha = beta = 0, gamma = 10, no KV split; run_benchmark.sh:67-81)
    merged = None
    if not args.no_gathered and args.workload != "c4":
        from fasttree_hip.planner import FastTreeParams, fasttree_preparation
        g = prob["hq"] // prob["hkv"]
        p2 = FastTreeParams()
        p2.set_values(0.0, 0.0, 10.0)
        p2.set_q_tile_sizes(list(prob["q_tiles"]))
        p2.set_kv_tile_sizes(list(prob["kv_tiles"]))
        p2.set_kv_group_num(g)
        aux2, assign2 = fasttree_preparation(prob["tree"], inp.KV_ptrs, prob["batch"], prob["hq"], prob["hkv"], 128,
                                             [81920, 81920], [0, 0], [0, 0], p2, device=device,
                                             kv_slot_map=inp.slot_map, launch_order=True)
        om = torch.empty_like(inp.Q)
        ts = []
        for i in range(13):
            flush_caches(clean=False)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fasttree_decode(inp.Q, inp.K_pool, inp.V_pool, om, *aux2, list(p2.TSQs), list(p2.TSKs), scale)
            e1.record()
            e1.synchronize()
            if i >= 3:
                ts.append(e0.elapsed_time(e1) * 1e3)
        merged = {"latency_us": statistics.median(ts), "merged_nodes": int(sum(assign2)),
                  "max_abs_vs_tree": float((om.float() - o.float()).abs().max())}
        del aux2

    # ---- CPU baseline: the reference's per-request gathered formulation with PyTorch ops on the host
    cpu = None
    if not args.no_cpu_baseline:
        cores = os.cpu_count() or 1
        threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        torch.set_num_threads(threads)
        qc, kc, vc = inp.Q.cpu(), inp.K_pool.cpu(), inp.V_pool.cpu()
        t = time.perf_counter()
        oracle.gathered_attention_torch(qc, kc, vc, inp.path_tokens, scale, requests=[0])
        one = time.perf_counter() - t
        n = max(2, min(prob["batch"], int(4.0 / max(one, 1e-4))))
        picks = [int(i * prob["batch"] / n) for i in range(n)]
        times = []
        for _ in range(3):
            t = time.perf_counter()
            oracle.gathered_attention_torch(qc, kc, vc, inp.path_tokens, scale, requests=picks)
            times.append(time.perf_counter() - t)
        cpu_us = statistics.median(times) * 1e6 * prob["batch"] / n
        cpu = {"value": cpu_us, "unit": "us", "cores": threads, "kind": "port",
               "sample": f"{n} of {prob['batch']} requests (evenly spaced), median of 3 passes, scaled to all requests"}

    result = {
        "metric": "tree-attention decode latency",
        "value": cold_med if parity["passed"] else None,
        "value_method": VALUE_METHOD,
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "device_warmup_ms": DEVICE_WARMUP_MS,
        "ms_per_step": wall_ms,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if prob["dtype"] == "fp16" else "bf16",
        "data": "synthetic",
        "config": {"workload": {"c1": "2-level tree 1x1024 + 16x128", "c2": "2-level tree 1x4096 + 64x256", "c3": "3-level tree N=[1,10,400] C=[4000,400,40]",
                                "c4": "2-level tree 1x512 + 2048x1024",
                                "c5": "irregular 5-level tree, seed 0"}[args.workload]
                   + f", {prob['hq']}q/{prob['hkv']}kv heads, head_dim 128, {prob['dtype']}, paged pool (page 1, shuffled), "
                   + f"{prob['batch']} requests", "planner_preset": args.preset,
                   "q_tiles": prob["q_tiles"], "vnodes": [int(x) for x in nums], "scratch_rows": int(rows)},
        "latency_us": {"cold_median": cold_med, "cold_p20": cold_p20, "cold_p80": cold_p80,
                       "cold_clean_median": statistics.median(cold_clean), "warm_median": warm_med},
        "effective_kv": {"algorithmic_bytes": prob["algo_bytes"], "GBps": prob["algo_bytes"] / (cold_med * 1e-6) / 1e9,
                         "hbm_frac": prob["algo_bytes"] / (cold_med * 1e-6) / 1e9 / HBM_PEAK_GBS,
                         "algorithmic_gflop": prob["algo_flops"] / 1e9},
        "per_launch_us": per_launch,
        "host_us_per_call": host_us,
        "roofline": roofline,
        "parity": parity,
        "gathered_hip_baseline": gathered,
        "speedup_vs_gathered": (gathered["latency_us"] / cold_med) if gathered else None,
        "all_merged_plan_baseline": merged,
        "cpu_baseline": cpu,
        "planner_ms": prob["plan_ms"],
    }
    print(json.dumps(result))
    if not parity["passed"]:
        log(f"bench.py: PARITY FAILED against the oracle ({parity}); the value is withheld")
        sys.exit(1)


if __name__ == "__main__":
    main()
