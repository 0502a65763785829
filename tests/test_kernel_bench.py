"""The kernel benchmark harness (the command lines of kernel_bench/benchmark.py,
tree_generation.py and run_benchmark.sh): argument surface and file formats on the CPU, one
small end-to-end run on the GPU."""
import os
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "fasttree-artifact_amd", "kernel_bench"))

import benchmark  # noqa: E402
import run_benchmark  # noqa: E402
import tree_generation  # noqa: E402
from fasttree_hip.kv_tree import generate_tree, retrive_from_file  # noqa: E402


def test_tree_generation_command_line_writes_the_tree_file(tmp_path):
    """-n / -l / -o as in kernel_bench/tree_generation.py:3-17; the file reads back as the
    generator's rows (format of kernel_bench/kv_tree_simple.py:50-64)."""
    path = tmp_path / "t.txt"
    tree_generation.main(["-n", "1,3,7", "-l", "50,20,9", "-o", str(path)])
    lines = path.read_text().split("\n")
    assert lines[0] == "11" and lines[1] == "-1 0 50 3"
    nodes = retrive_from_file(str(path))
    rows = generate_tree([1, 3, 7], [50, 20, 9])
    assert [[n.parent, n.id, n.seqlen, n.num_children] for n in nodes] == rows
    with pytest.raises(SystemExit):
        tree_generation.main(["-n", "1,3", "-o", str(path)])
    tree_generation.main(["--irregular_seed", "1", "-o", str(path)])
    assert len(retrive_from_file(str(path))) > 5


def test_benchmark_options_and_defaults_follow_the_reference():
    """kernel_bench/benchmark.py:241-275: same option names and defaults; the tile and threshold
    defaults are resolved in main() so that --mi355x can replace them."""
    args = benchmark.build_parser().parse_args(["--load_file_path", "x.txt"])
    assert (args.alpha, args.beta, args.gamma) == (0.66, 0.33, 0.1)
    assert args.kv_tile_size_per_phase == "32,32"
    assert (args.num_qo_heads, args.num_kv_heads, args.head_dim) == (32, 32, 128)
    assert args.choice == "all" and args.signature is None and args.fasttree_heuristic_path is None and args.profile is False
    assert args.q_tile_size_per_phase is None and args.para_threshs1 is None and args.para_threshs2 is None
    assert args.kv_split_sizes is None
    assert benchmark.planner_options(args) == ([64, 16], [32, 32], [1024, 128], [132, 528], [132, 132])
    gqa = ["--load_file_path", "x.txt", "--num_qo_heads", "32", "--num_kv_heads", "8"]
    assert benchmark.planner_options(benchmark.build_parser().parse_args(gqa + ["--mi355x"])) == (
        [16, 4], [32, 32], [1024, 256], [256, 1024], [256, 256])
    # an explicit option wins over --mi355x
    explicit = benchmark.build_parser().parse_args(gqa + ["--mi355x", "--kv_split_sizes", "512,64", "--para_threshs2", "1,2"])
    assert benchmark.planner_options(explicit) == ([16, 4], [32, 32], [512, 64], [256, 1024], [1, 2])
    assert benchmark.build_parser().parse_args(["--load_file_path", "x.txt", "--choice", "DeFT"]).choice == "DeFT"
    with pytest.raises(SystemExit):
        benchmark.build_parser().parse_args(["--load_file_path", "x.txt", "--choice", "flashinfer"])
    with pytest.raises(SystemExit):
        benchmark.build_parser().parse_args([])


def test_sweep_lists_and_table():
    """The tree list and head configurations of kernel_bench/run_benchmark.sh:5-27, its tile
    choice per GQA ratio (:46-53), and the normalised table (plot_norm_perf.py:27)."""
    assert len(run_benchmark.NODES_CONTEXTS) == 15 and run_benchmark.QK_HEADS == [(16, 1), (32, 8), (32, 32)]
    for nodes, contexts in run_benchmark.NODES_CONTEXTS:
        assert len(nodes.split(",")) == len(contexts.split(",")) and nodes.startswith("1,")
    assert [run_benchmark.reference_q_tiles(g) for g in (1, 4, 16, 8)] == ["64,16", "16,4", "4,1", "8,2"]


def test_sweep_table_is_normalised_to_the_best_engine(tmp_path):
    row = dict(tree="1,2 / 8,8", heads="32/8", preset="mi355x", flash_attn=0.4, naive=0.2, deft=0.125, cascade=0.2, no_greedy=0.1,
               fasttree=0.05, check=True, deft_check=True, max_abs=1e-4, mean_abs=1e-5)
    path = tmp_path / "r.md"
    run_benchmark.write_table([row], str(path))
    body = path.read_text().split("\n")[2]
    assert "| 8.00 |" in body and "0.12 / 0.25 / 0.40 / 0.25 / 0.50 / 1.00" in body and "passed" in body
    row["deft_check"] = False
    run_benchmark.write_table([row], str(path))
    assert "FAILED" in path.read_text().split("\n")[2]


def test_plot_script_reads_the_sweep_table_and_draws_it(tmp_path):
    """plot_norm_perf.py takes the table run_benchmark.py writes: one row per case of the chosen
    preset, every engine column present, and a picture comes out."""
    import plot_norm_perf
    rows = [dict(tree=f"1,{n} / 8,8", heads=h, preset=p, flash_attn=0.4, naive=0.2, deft=0.125, cascade=0.2, no_greedy=0.1,
                 fasttree=0.05, check=True, deft_check=True, max_abs=1e-4, mean_abs=1e-5)
            for n in (2, 4) for h in ("16/1", "32/8") for p in ("reference", "mi355x")]
    table = tmp_path / "r.md"
    run_benchmark.write_table(rows, str(table))
    got = plot_norm_perf.read_table(str(table), "mi355x")
    assert len(got) == 4 and all(r["preset"] == "mi355x" for r in got)
    assert all(column in got[0] for column, _, _ in plot_norm_perf.ENGINES)
    assert float(got[0]["tree ms"]) == 0.05 and float(got[0]["DeFT ms"]) == 0.125
    out = tmp_path / "r.png"
    assert plot_norm_perf.main(["--input", str(table), "--preset", "mi355x", "--output", str(out)]) == 0
    assert out.stat().st_size > 10000


def test_deft_schedule_partitions_the_flattened_tree():
    """kernel_bench/DeFT.py:14-55 by hand on a small tree: depth-first token order, subtrees of
    `subtree_len` tokens, a node cut wherever a subtree is full; and on the trees of the
    planner's fixtures every request still attends every token of its path exactly once."""
    import deft_schedule
    from fasttree_hip.kv_tree import assign_requests, kv_prefix_sums, nodes_from_rows, root_path
    # root 10 tokens; children a (7 tokens, leaves a1 3, a2 4) and b (5 tokens, leaf)
    tree = nodes_from_rows([[-1, 0, 10, 2], [0, 1, 7, 2], [1, 2, 3, 0], [1, 3, 4, 0], [0, 4, 5, 0]])
    batch = assign_requests(tree)
    assert batch == 3
    subtrees = deft_schedule.group_subtrees(tree, 8)
    # depth-first order: 0 (10), 1 (7), 2 (3), 3 (4), 4 (5) = 29 tokens -> 8, 8, 8, 5
    assert subtrees == [[(0, 0, 8)], [(0, 8, 10), (1, 0, 6)], [(1, 6, 7), (2, 0, 3), (3, 0, 4)], [(4, 0, 5)]]
    assert deft_schedule.group_subtrees(tree, 10)[:2] == [[(0, 0, 10)], [(1, 0, 7), (2, 0, 3)]]   # a node that ends with its subtree
    ptrs = kv_prefix_sums(tree)
    lists = deft_schedule.deft_lists(tree, ptrs, batch, group=4, subtree_len=8, block_rows=8)      # two requests per vnode
    # the root's pieces are attended by all three requests in chunks of two: (0,1) and (2,)
    assert lists["kv_offs"][:2].tolist() == [0, 0] and lists["kv_lens"][:2].tolist() == [8, 8]
    assert lists["q_lens"][:2].tolist() == [2, 1] and lists["q_entries"][:3].tolist() == [0, 1, 2]
    assert lists["prog_table"].tolist() == [[0, 2, 0, 0], [2, 5, 0, 0], [5, 8, 0, 0], [8, 9, 0, 0]]
    from cases import PLANNER_CASES
    from helpers import run_planner
    for name in ("c1", "c3", "c5_seed0", "rand03", "rand17"):
        case = next(c for c in PLANNER_CASES if c["name"] == name)
        tree, ptrs, batch, plan, params, _ = run_planner(case)
        group = case["Hq"] // case["Hkv"]
        lists = deft_schedule.deft_lists(tree, ptrs, batch, group)
        assert (lists["q_lens"] * group <= 128).all() and (lists["kv_lens"] > 0).all() and (lists["kv_lens"] <= 128).all()
        t = lists["prog_table"]
        assert t[0, 0] == 0 and t[-1, 1] == len(lists["kv_offs"]) and (t[1:, 0] == t[:-1, 1]).all()
        assert len(t) == -(-int(ptrs[-1]) // 128)
        seen = [[] for _ in range(batch)]
        for v in range(len(lists["kv_offs"])):
            for i in range(lists["q_lens"][v]):
                r = lists["q_entries"][lists["q_offs"][v] + i]
                seen[r].extend(range(lists["kv_offs"][v], lists["kv_offs"][v] + lists["kv_lens"][v]))
        leaves = [i for i, n in enumerate(tree) if n.num_children == 0]
        for r in range(batch):
            want = [t for n in root_path(tree, leaves[r]) for t in range(ptrs[n], ptrs[n + 1])]
            assert sorted(seen[r]) == sorted(want)
            rows = lists["req_entries"][lists["req_offs"][r]: lists["req_offs"][r] + lists["req_lens"][r]]
            assert all(lists["q_entries"][x] == r for x in rows)
        assert lists["req_lens"].sum() == len(lists["q_entries"])


@pytest.mark.gpu
def test_benchmark_runs_both_engines_and_checks_them(tmp_path, capsys):
    import torch
    assert torch.cuda.is_available()
    path = tmp_path / "t.txt"
    tree_generation.main(["-n", "1,4,24", "-l", "300,70,33", "-o", str(path)])
    plan_path = tmp_path / "plan.txt"
    res = benchmark.main(benchmark.build_parser().parse_args(
        ["--load_file_path", str(path), "--num_qo_heads", "32", "--num_kv_heads", "8", "--mi355x",
         "--fasttree_heuristic_path", str(plan_path)]))
    out = capsys.readouterr().out
    assert "flash attn time:" in out and "fasttree attn time:" in out and "fasttree attn Check passed!" in out
    assert "DeFT attn time:" in out and "DeFT attn Check passed!" in out and res["deft_check"]
    assert "parallelisms:" in out  # the planner's own lines, as the reference prints them
    assert res["check"] and res["max_abs"] <= 2e-3 and res["worst_request_mean_abs"] <= 1e-3
    assert plan_path.read_text().startswith("Node 0: parent -1, assignment 0\n")
    res = benchmark.main(benchmark.build_parser().parse_args(
        ["--load_file_path", str(path), "--choice", "fasttree", "--alpha", "0", "--beta", "0", "--gamma", "10",
         "--kv_split_sizes", "81920,81920", "--signature", "fasttree 10", "--quiet", "--profile"]))
    assert list(res) == ["fasttree 10"]
