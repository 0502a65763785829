"""The reference's kernel sweep (kernel_bench/run_benchmark.sh:5-92) in one process, with the table
its parse_output.py / plot_norm_perf.py derive: 15 level-regular trees x 3 head configurations;
per case the gathered decode without sharing ("flash attn"), the tree decode, the two ablations
of the tree decode (gamma = 10 with one KV split: every request its own full path, "naive";
gamma = -10: never merge, "w/o greedy"), multi-level cascade attention ("cascade": every tree
node one batched attention over its own KV, merged per request -- bench_cascade.py here, the
plan / run calls of the wrapper the reference measures with FlashInfer,
kernel_bench/bench_cascade.py and run_benchmark.sh:83-88), and DeFT-Flatten (subtrees of 128 tokens of the depth-first token
order, one block per subtree with a mask word per token, kernel_bench/DeFT.py) on its own kernel.

    python run_benchmark.py --out sweep --preset mi355x [--cases 0,8,9] [--heads "32 8"]

Writes ``<out>/trees/*.txt``, ``<out>/outputs/*.txt`` (``outputs_<preset>`` with ``--preset both``;
the lines benchmark.py prints, under the file names the reference's parse_output.py reads) and
``<out>/results.md``: milliseconds per engine, the speed-up of the tree decode over the gathered
decode, and performance normalised to the best engine of the row
(kernel_bench/plot_norm_perf.py:27).
"""
import argparse
import contextlib
import io
import math
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

import bench_cascade  # noqa: E402
import benchmark  # noqa: E402
import tree_generation  # noqa: E402

# (kernel_bench/run_benchmark.sh:5-21)
NODES_CONTEXTS = [
    ("1,2,64", "8,256,32"),
    ("1,4,256", "8,256,32"),
    ("1,4,8,256", "8,256,256,32"),
    ("1,256", "256,32"),
    ("1,1024", "2048,32"),
    ("1,16,64", "1024,256,32"),
    ("1,4,16,512", "1024,256,128,32"),
    ("1,4,16,64,256,1024", "256,8,256,64,32,256"),
    ("1,10", "4000,400"),
    ("1,2,4,8,16,32,64,128,1024", "16,16,16,16,16,16,16,16,16"),
    ("1,2,4,8,16,32,64,128,1024", "256,128,64,16,16,16,16,16,16"),
    ("1,8,16,32,64,128,1024", "256,128,64,16,16,16,16"),
    ("1,8,16,32,64,256,1024", "256,128,64,16,16,16,16"),
    ("1,16,32,64,128,1024", "256,128,64,16,16,16"),
    ("1,16,32,64,256,1024", "256,128,64,16,16,16"),
]
QK_HEADS = [(16, 1), (32, 8), (32, 32)]  # (kernel_bench/run_benchmark.sh:23-27)


def reference_q_tiles(group):
    """The sweep's tile choice per GQA ratio (kernel_bench/run_benchmark.sh:46-53)."""
    return {1: "64,16", 4: "16,4", 16: "4,1"}.get(group, f"{max(1, 64 // group)},{max(1, 16 // group)}")


def run_case(out_dir, nodes, contexts, q_heads, k_heads, preset, log=print, extra=(), outputs="outputs"):
    tree = f"nc_{nodes}_{contexts}.txt"
    tree_path = os.path.join(out_dir, "trees", tree)
    if not os.path.exists(tree_path):
        tree_generation.main(["-n", nodes, "-l", contexts, "-o", tree_path])
    # (the file name the reference's parse_output.py expects, kernel_bench/parse_output.py:93)
    out_path = os.path.join(out_dir, outputs, f"nc_{nodes}_{contexts}_qk_{q_heads}_{k_heads}.txt")
    base = ["--load_file_path", tree_path, "--num_qo_heads", str(q_heads), "--num_kv_heads", str(k_heads)]
    if preset == "mi355x":
        base += ["--mi355x"]
    else:
        base += ["--q_tile_size_per_phase", reference_q_tiles(q_heads // k_heads)]
    base += list(extra)
    runs = [
        ("all", base + ["--choice", "all"]),
        ("naive", base + ["--choice", "fasttree", "--alpha", "0", "--beta", "0", "--gamma", "10",
                          "--kv_split_sizes", "81920,81920", "--signature", "fasttree 10"]),
        ("no_greedy", base + ["--choice", "fasttree", "--alpha", "0", "--beta", "0", "--gamma", "-10",
                              "--signature", "fasttree -10"]),
    ]
    row = {"tree": f"{nodes} / {contexts}", "heads": f"{q_heads}/{k_heads}", "preset": preset}
    with open(out_path, "w") as fh:
        for tag, argv in runs:
            text = io.StringIO()
            with contextlib.redirect_stdout(text):
                res = benchmark.main(benchmark.build_parser().parse_args(argv))
            fh.write(text.getvalue())
            if tag == "all":
                row["flash_attn"] = res.get("flash attn")
                row["fasttree"] = res.get("fasttree attn")
                row["deft"] = res.get("DeFT attn")
                row["deft_check"] = res.get("deft_check")
                row["check"] = res.get("check")
                row["max_abs"] = res.get("max_abs")
                row["mean_abs"] = res.get("worst_request_mean_abs")
                row["modelled_us"] = res.get("stage1_modelled_us")
                row["measured_us"] = res.get("stage1_measured_us")
            else:
                row[tag] = next(iter(v for k, v in res.items() if k.startswith("fasttree")), None)
        text = io.StringIO()
        with contextlib.redirect_stdout(text):
            row["cascade"] = bench_cascade.main(["--node_num_per_level", nodes, "--node_seqlen_per_level", contexts,
                                                 "--num_qo_heads", str(q_heads), "--num_kv_heads", str(k_heads)])["cascade"]
        fh.write(text.getvalue())
    log(f"{row['tree']:60s} {row['heads']:6s} {preset:9s} gathered {row['flash_attn']:.4f} ms  tree {row['fasttree']:.4f} ms  "
        f"naive {row['naive']:.4f}  w/o greedy {row['no_greedy']:.4f}  cascade {row['cascade']:.4f}  DeFT {row['deft']:.4f}  "
        f"check {row['check']} / {row['deft_check']}  max abs {row['max_abs']:.1e}")
    return row


def write_table(rows, path):
    engines = ["flash_attn", "naive", "deft", "cascade", "no_greedy", "fasttree"]
    with open(path, "w") as fh:
        fh.write("| tree (nodes / tokens per level) | q/kv heads | preset | gathered ms | tree, naive ms | DeFT ms | cascade ms | tree, w/o greedy ms | tree ms | "
                 "speed-up over gathered | normalised: gathered / naive / DeFT / cascade / w/o greedy / tree | allclose 1e-2 | max abs | worst request mean abs |\n")
        fh.write("|---|---|---|---|---|---|---|---|---|---|---|---|---|---|\n")
        for r in rows:
            best = min(r[e] for e in engines)
            norm = " / ".join(f"{best / r[e]:.2f}" for e in engines)
            fh.write(f"| {r['tree']} | {r['heads']} | {r['preset']} | {r['flash_attn']:.4f} | {r['naive']:.4f} | {r['deft']:.4f} | {r['cascade']:.4f} | {r['no_greedy']:.4f} | "
                     f"{r['fasttree']:.4f} | {r['flash_attn'] / r['fasttree']:.2f} | {norm} | {'passed' if r['check'] and r['deft_check'] else 'FAILED'} | "
                     f"{r['max_abs']:.1e} | {r['mean_abs']:.1e} |\n")
        fh.write("\n")
        for preset in sorted({r["preset"] for r in rows}):
            part = [r for r in rows if r["preset"] == preset]
            geo = math.exp(sum(math.log(r["flash_attn"] / r["fasttree"]) for r in part) / len(part))
            best = sum(1 for r in part if r["fasttree"] <= 1.05 * min(r[e] for e in engines))
            fh.write(f"Preset `{preset}`: {len(part)} cases, geometric-mean speed-up of the tree decode over the gathered "
                     f"decode {geo:.2f}x; the tree decode is the fastest engine (within 5 %) in {best} of them; "
                     f"{sum(1 for r in part if not (r['check'] and r['deft_check']))} failed the allclose check (tree decode or DeFT).\n\n")


def write_model_check(rows, path):
    """The launch schedule's modelled duration of the first-stage launch beside the measured one
    (warm, per launch of a run of launches queued back to back: the kernel plus the gap before the next one), for the
    cases whose lists were arranged as block programs."""
    rows = [r for r in rows if r.get("modelled_us") is not None]
    with open(path, "w") as fh:
        fh.write("| tree (nodes / tokens per level) | q/kv heads | modelled us | measured us | modelled / measured |\n|---|---|---|---|---|\n")
        for r in rows:
            fh.write(f"| {r['tree']} | {r['heads']} | {r['modelled_us']:.1f} | {r['measured_us']:.1f} | {r['modelled_us'] / r['measured_us']:.2f} |\n")
        if rows:
            ratios = [r["modelled_us"] / r["measured_us"] for r in rows]
            geo = math.exp(sum(math.log(x) for x in ratios) / len(ratios))
            inside = sum(1 for x in ratios if 0.8 <= x <= 1.2)
            fh.write(f"\n{len(rows)} launches: modelled / measured between {min(ratios):.2f} and {max(ratios):.2f}, geometric mean "
                     f"{geo:.2f}; {inside} within 20 % of the measured time.\n")


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="sweep")
    ap.add_argument("--preset", default="mi355x", choices=["reference", "mi355x", "both"])
    ap.add_argument("--cases", default=None, help="comma-separated indices into the tree list (default: all)")
    ap.add_argument("--heads", default=None, help='one head configuration, e.g. "32 8" (default: all three)')
    ap.add_argument("--extra", default="", help="further benchmark.py options for every run, as one string")
    args = ap.parse_args(argv)
    presets = ["reference", "mi355x"] if args.preset == "both" else [args.preset]
    outputs = {p: "outputs" if len(presets) == 1 else f"outputs_{p}" for p in presets}
    for sub in ["trees", *outputs.values()]:
        os.makedirs(os.path.join(args.out, sub), exist_ok=True)
    cases = range(len(NODES_CONTEXTS)) if args.cases is None else [int(x) for x in args.cases.split(",")]
    heads = QK_HEADS if args.heads is None else [tuple(int(x) for x in args.heads.split())]
    rows = []
    for c in cases:
        nodes, contexts = NODES_CONTEXTS[c]
        for q_heads, k_heads in heads:
            for preset in presets:
                rows.append(run_case(args.out, nodes, contexts, q_heads, k_heads, preset,
                                     log=lambda *a: print(*a, flush=True), extra=args.extra.split(),
                                     outputs=outputs[preset]))
                write_table(rows, os.path.join(args.out, "results.md"))
                write_model_check(rows, os.path.join(args.out, "model_check.md"))
    failed = [r for r in rows if not (r["check"] and r["deft_check"])]
    print(f"{len(rows)} cases, {len(failed)} failed the allclose check", flush=True)
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
