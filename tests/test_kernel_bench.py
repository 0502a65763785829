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
    with pytest.raises(SystemExit):
        benchmark.build_parser().parse_args(["--load_file_path", "x.txt", "--choice", "DeFT"])
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
    row = dict(tree="1,2 / 8,8", heads="32/8", preset="mi355x", flash_attn=0.4, naive=0.2, node_wise=0.2, no_greedy=0.1, fasttree=0.05,
               check=True, max_abs=1e-4, mean_abs=1e-5)
    path = tmp_path / "r.md"
    run_benchmark.write_table([row], str(path))
    body = path.read_text().split("\n")[2]
    assert "| 8.00 |" in body and "0.12 / 0.25 / 0.25 / 0.50 / 1.00" in body and "passed" in body


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
    assert "parallelisms:" in out  # the planner's own lines, as the reference prints them
    assert res["check"] and res["max_abs"] <= 2e-3 and res["worst_request_mean_abs"] <= 1e-3
    assert plan_path.read_text().startswith("Node 0: parent -1, assignment 0\n")
    res = benchmark.main(benchmark.build_parser().parse_args(
        ["--load_file_path", str(path), "--choice", "fasttree", "--alpha", "0", "--beta", "0", "--gamma", "10",
         "--kv_split_sizes", "81920,81920", "--signature", "fasttree 10", "--quiet", "--profile"]))
    assert list(res) == ["fasttree 10"]
