"""Kernel micro-benchmark with the command line of kernel_bench/benchmark.py:241-275.

    python benchmark.py --load_file_path trees/c3.txt --num_qo_heads 32 --num_kv_heads 8 \\
        --q_tile_size_per_phase 16,4 --choice all

Engines (``--choice``): ``fasttree`` is the tree decode (planner + the two HIP stages);
``flash_attn`` is the decode without prefix sharing over the per-request gathered cache
``[B, max_seqlen, Hkv, D]`` (the layout of kernel_bench/flash_attn_wrap.py:36-70), here a HIP
kernel of this library, and it is the result the tree decode is checked against with the
reference's criterion ``allclose(rtol=1e-2, atol=1e-2)`` (kernel_bench/benchmark.py:216-220).
``DeFT`` is DeFT-Flatten as the reference benchmarks it (kernel_bench/DeFT.py, benchmark.py:180-211):
the depth-first token order cut into subtrees of 128 tokens, one thread block per (subtree, kv
head) over the subtree's whole query set with a 64-bit mask word per token and group of 64
requests, reading the per-request gathered cache -- this library's ``DeFT.py`` on its own HIP
kernel; it is checked against the gathered decode like the tree decode.  ``DeFT_schedule`` runs the
same partition through the *tree* kernels instead (one vnode per node piece, ``deft_schedule.py``;
kept for comparison, not part of ``all``).  The reference's other engines (SGLang Triton,
FlashInfer) are Triton / CUDA libraries and have no counterpart here.

Timing follows the method of ``triton.testing.do_bench`` as the reference calls it
(kernel_bench/benchmark.py:35,59): per-call device events, a 256 MB buffer cleared before every
call, a repetition count sized for about 100 ms, the median reported in milliseconds.
``--mi355x`` replaces the H100 defaults of the query tiles (64,16, right for 32/32 heads only), of
the parallelism thresholds and of the KV split sizes with the ones for MI355X: tiles of 64 // g
and 16 // g requests, as the reference's sweep picks them per GQA ratio
(kernel_bench/run_benchmark.sh:46-53), thresholds for 256 compute units instead of 132, and KV
splits of 1024,256 instead of 1024,128 tokens; explicit options win over it.  It also asks the
planner for its lists arranged as block programs for the part (``launch_order=True``) instead of in
the reference's order.
"""
import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from fasttree_hip import planner as _planner  # noqa: E402
from fasttree_hip.decode import fasttree_decode, fasttree_decode_stage1, gathered_decode  # noqa: E402
from fasttree_hip.inputs import qkv_preparation  # noqa: E402
from fasttree_hip.kv_tree import retrive_from_file  # noqa: E402
from fasttree_hip.planner import FastTreeParams, fasttree_preparation  # noqa: E402
from deft_schedule import deft_preparation  # noqa: E402
from DeFT import DeFT_decode, DeFT_preparation  # noqa: E402

QUANTILES = [0.5, 0.2, 0.8]


def do_bench(fn, quantiles=QUANTILES, warmup=25, rep=100):
    """Milliseconds per call at the given quantiles; cold L2 (a 256 MB buffer is cleared before
    every call), one event pair per call."""
    fn()
    torch.cuda.synchronize()
    cache = torch.empty(256 << 20, dtype=torch.int8, device="cuda")
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        cache.zero_()
        fn()
    end.record()
    torch.cuda.synchronize()
    estimate = start.elapsed_time(end) / 5
    n_warmup = max(1, int(warmup / estimate))
    n_repeat = max(1, int(rep / estimate))
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for _ in range(n_warmup):
        fn()
    for i in range(n_repeat):
        cache.zero_()
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([s.elapsed_time(e) for s, e in zip(starts, ends)], dtype=torch.float64)
    return torch.quantile(times, torch.tensor(quantiles, dtype=torch.float64)).tolist()


def planner_options(args):
    """Query tiles, KV tiles, KV split sizes and the two threshold pairs as lists of int: the
    options given, else the reference's defaults (kernel_bench/benchmark.py:246-254), else with
    --mi355x the ones for MI355X."""
    group = args.num_qo_heads // args.num_kv_heads
    defaults = dict(q_tile_size_per_phase="64,16", kv_split_sizes="1024,128", para_threshs1="132,528", para_threshs2="132,132")
    if args.mi355x:
        defaults = dict(q_tile_size_per_phase=f"{max(1, 64 // group)},{max(1, 16 // group)}", kv_split_sizes="1024,256",
                        para_threshs1="256,1024", para_threshs2="256,256")
    ints = lambda text: list(map(int, text.split(",")))
    return (ints(args.q_tile_size_per_phase or defaults["q_tile_size_per_phase"]), ints(args.kv_tile_size_per_phase),
            ints(args.kv_split_sizes or defaults["kv_split_sizes"]), ints(args.para_threshs1 or defaults["para_threshs1"]),
            ints(args.para_threshs2 or defaults["para_threshs2"]))


def main(args):
    num_qo_heads, num_kv_heads, head_dim = args.num_qo_heads, args.num_kv_heads, args.head_dim
    group = num_qo_heads // num_kv_heads
    dtype = torch.float16
    Q_TILE_SIZE_PER_PHASE, KV_TILE_SIZE_PER_PHASE, KV_SPLIT_SIZES, para_threshs1, para_threshs2 = planner_options(args)

    params = FastTreeParams()
    params.set_values(args.alpha, args.beta, args.gamma)
    params.set_q_tile_sizes(Q_TILE_SIZE_PER_PHASE)
    params.set_kv_tile_sizes(KV_TILE_SIZE_PER_PHASE)
    params.set_kv_group_num(group)

    tree_info = retrive_from_file(args.load_file_path)
    Q, K_cache, V_cache, cache_seqlens, K_tree_tensor, V_tree_tensor, KV_ptrs = qkv_preparation(
        tree_info, num_qo_heads, num_kv_heads, head_dim, "cuda", dtype)
    batch_size = Q.shape[0]
    sm_scale = 1.0 / (head_dim ** 0.5)
    results = {}

    def run_and_bench(func, name):
        if args.signature:
            name = args.signature
        out = func()
        ms, _, _ = do_bench(func, quantiles=QUANTILES)
        if args.profile:
            # one more call between the profiler's start and stop marks, inside a named range
            # (kernel_bench/benchmark.py:12-24,60-63 does this with cudaProfilerStart/Stop)
            torch.cuda.synchronize()
            torch.cuda.profiler.start()
            torch.cuda.nvtx.range_push(name)
            func()
            torch.cuda.synchronize()
            torch.cuda.nvtx.range_pop()
            torch.cuda.profiler.stop()
        print(f"{name} time:", ms, flush=True)
        results[name] = ms
        return out

    out_flash_attn = None
    out_tree_attn = None

    if args.choice in ["flash_attn", "all"]:
        out_gathered = torch.empty(batch_size, num_qo_heads, head_dim, device="cuda", dtype=dtype)
        kv_split = 512
        nsplit = (K_cache.shape[1] + kv_split - 1) // kv_split
        mid_o = torch.empty((batch_size * nsplit, num_qo_heads, head_dim), dtype=torch.float32, device="cuda")
        mid_lse = torch.empty((batch_size * nsplit, num_qo_heads), dtype=torch.float32, device="cuda")

        def call_gathered():
            gathered_decode(Q, K_cache, V_cache, cache_seqlens, out_gathered, sm_scale, kv_split, mid_o, mid_lse)
            return out_gathered

        out_flash_attn = run_and_bench(call_gathered, "flash attn").cpu()

    if args.choice in ["fasttree", "all"]:
        _planner.VERBOSE = not args.quiet
        fasttree_aux, node_assignment = fasttree_preparation(
            tree_info, KV_ptrs, batch_size, num_qo_heads, num_kv_heads, head_dim,
            KV_SPLIT_SIZES, para_threshs1, para_threshs2, params, launch_order=args.mi355x)
        if args.fasttree_heuristic_path:
            with open(args.fasttree_heuristic_path, "w") as file:
                for i in range(len(tree_info)):
                    file.write(f"Node {i}: parent {tree_info[i].parent}, assignment {node_assignment[i]}\n")
        out_tree = torch.empty(batch_size, num_qo_heads, head_dim, device="cuda", dtype=dtype)
        # (the tiles the planner ended with; they differ from the command line's only when its
        # second pass collapsed the phases, kernel_bench/fasttree.py:181-186)
        q_tiles, kv_tiles = list(params.TSQs), list(params.TSKs)

        def call_tree_attn():
            fasttree_decode(Q, K_tree_tensor, V_tree_tensor, out_tree, *fasttree_aux, q_tiles, kv_tiles, sm_scale)
            return out_tree

        out_tree_attn = run_and_bench(call_tree_attn, "fasttree attn").cpu()
        modelled = getattr(fasttree_aux[11], "modelled_us", None)
        if modelled is not None and not args.signature:
            # what the launch schedule's model expects of the first-stage launch beside what it takes: the
            # launches run back to back behind a filler that keeps the device busy while the host queues them
            # (so the host's call rate and the cost of an event between two launches stay out of the figure;
            # warm caches, as the model's constants were measured), timed in runs of twenty
            def call_stage1():
                fasttree_decode_stage1(Q, K_tree_tensor, V_tree_tensor, *fasttree_aux[:6], sm_scale, fasttree_aux[9],
                                       fasttree_aux[10], fasttree_aux[11], fasttree_aux[12], q_tiles, kv_tiles)

            for _ in range(20):
                call_stage1()
            filler = torch.empty(int(256e6), dtype=torch.int8, device="cuda")
            runs, per_run = 5, 20
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(runs + 1)]
            torch.cuda.synchronize()
            for _ in range(32):
                filler.zero_()
            for _ in range(per_run):                    # (these also write the filler's dirty lines back)
                call_stage1()
            marks[0].record()
            for i in range(runs):
                for _ in range(per_run):
                    call_stage1()
                marks[i + 1].record()
            torch.cuda.synchronize()
            measured = torch.tensor([a.elapsed_time(b) for a, b in zip(marks, marks[1:])]).median().item() * 1e3 / per_run
            print(f"fasttree stage 1: modelled {modelled:.1f} us, measured {measured:.1f} us per launch back to back (warm), "
                  f"{fasttree_aux[11].num_programs} programs on {fasttree_aux[11].block_slots} block slots", flush=True)
            results["stage1_modelled_us"], results["stage1_measured_us"] = float(modelled), float(measured)

    out_deft_attn = None
    if args.choice in ["DeFT", "all"]:
        subtree_len, mask_len = 128, 64  # (kernel_bench/benchmark.py:183-184)
        deft_aux = DeFT_preparation(tree_info, K_cache, subtree_len, mask_len, num_qo_heads, head_dim)
        out_deft = torch.empty(batch_size, num_qo_heads, head_dim, device="cuda", dtype=dtype)
        k_flat = K_cache.view(-1, K_cache.shape[-2], K_cache.shape[-1])
        v_flat = V_cache.view(-1, V_cache.shape[-2], V_cache.shape[-1])

        def call_deft_attn():
            DeFT_decode(Q, k_flat, v_flat, out_deft, *deft_aux, Q_TILE_SIZE_PER_PHASE[0], KV_TILE_SIZE_PER_PHASE[0],
                        sm_scale, mask_len)
            return out_deft

        out_deft_attn = run_and_bench(call_deft_attn, "DeFT attn").cpu()

    if args.choice == "DeFT_schedule":
        sched_aux = deft_preparation(tree_info, KV_ptrs, batch_size, num_qo_heads, num_kv_heads, head_dim, 128)
        out_sched = torch.empty(batch_size, num_qo_heads, head_dim, device="cuda", dtype=dtype)

        def call_deft_schedule():
            fasttree_decode(Q, K_tree_tensor, V_tree_tensor, out_sched, *sched_aux, [1, 1], [32, 32], sm_scale)
            return out_sched

        run_and_bench(call_deft_schedule, "DeFT schedule")

    if out_flash_attn is not None and out_deft_attn is not None:
        ok = torch.allclose(out_flash_attn, out_deft_attn, rtol=1e-2, atol=1e-2)
        print("DeFT attn Check passed!" if ok else "DeFT attn Check failed!", flush=True)
        results["deft_check"] = bool(ok)

    if out_flash_attn is not None and out_tree_attn is not None:
        ok = torch.allclose(out_flash_attn, out_tree_attn, rtol=1e-2, atol=1e-2)
        print("fasttree attn Check passed!" if ok else "fasttree attn Check failed!", flush=True)
        err = (out_flash_attn.float() - out_tree_attn.float()).abs()
        results["max_abs"] = err.max().item()
        results["worst_request_mean_abs"] = err.mean(dim=(1, 2)).max().item()
        results["check"] = bool(ok)
        print(f"max abs difference: {results['max_abs']:.3e}, worst request mean abs: "
              f"{results['worst_request_mean_abs']:.3e}", flush=True)
    return results


def build_parser():
    parser = argparse.ArgumentParser()
    parser.add_argument("--load_file_path", type=str, required=True)
    parser.add_argument("--alpha", type=float, default=0.66)
    parser.add_argument("--beta", type=float, default=0.33)
    parser.add_argument("--gamma", type=float, default=0.1)
    parser.add_argument("--q_tile_size_per_phase", type=str, default=None, help="default 64,16")
    parser.add_argument("--kv_tile_size_per_phase", type=str, default="32,32")
    parser.add_argument("--kv_split_sizes", type=str, default=None, help="default 1024,128")
    parser.add_argument("--para_threshs1", type=str, default=None, help="default 132,528")
    parser.add_argument("--para_threshs2", type=str, default=None, help="default 132,132")
    parser.add_argument("--fasttree_heuristic_path", type=str, default=None)
    parser.add_argument("--num_qo_heads", type=int, default=32)
    parser.add_argument("--num_kv_heads", type=int, default=32)
    parser.add_argument("--head_dim", type=int, default=128)
    parser.add_argument("--signature", type=str, default=None)
    parser.add_argument("--choice", type=str, choices=["flash_attn", "fasttree", "DeFT", "DeFT_schedule", "all"], default="all")
    parser.add_argument("--profile", action="store_true", default=False)
    parser.add_argument("--mi355x", action="store_true", default=False,
                        help="query tiles, parallelism thresholds and KV split sizes for MI355X instead of the H100 defaults, "
                             "and the planner's lists arranged as block programs for the part")
    parser.add_argument("--quiet", action="store_true", default=False, help="do not print the planner's lines")
    return parser


if __name__ == "__main__":
    main(build_parser().parse_args())
