"""Writes a level-regular tree file: the command line of kernel_bench/tree_generation.py:3-17,100-112.

    python tree_generation.py -n 1,10,400 -l 4000,400,40 -o trees/c3.txt
    python tree_generation.py --irregular_seed 0 -o trees/c5_seed0.txt

The file format is the one ``retrive_from_file`` reads (kernel_bench/kv_tree_simple.py:50-64).
``--irregular_seed`` (not in the reference) writes a seeded five-level irregular tree instead.
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from fasttree_hip.kv_tree import generate_irregular_tree, generate_tree, save_tree  # noqa: E402


def parse_args(argv=None):
    p = argparse.ArgumentParser(description="Generate a tree from per-level node counts and sequence lengths.")
    p.add_argument("-n", "--layer_sizes", type=str, default=None, help="node counts per level, e.g. 1,2,4")
    p.add_argument("-l", "--layer_lengths", type=str, default=None, help="sequence lengths per level, e.g. 128,64,64")
    p.add_argument("-o", "--output_file", type=str, required=True)
    p.add_argument("--irregular_seed", type=int, default=None, help="seeded irregular tree instead of a regular one")
    return p.parse_args(argv)


def main(argv=None):
    args = parse_args(argv)
    if args.irregular_seed is not None:
        rows = generate_irregular_tree(args.irregular_seed)
    else:
        if args.layer_sizes is None or args.layer_lengths is None:
            raise SystemExit("-n/--layer_sizes and -l/--layer_lengths are required for a regular tree")
        rows = generate_tree(list(map(int, args.layer_sizes.split(","))), list(map(int, args.layer_lengths.split(","))))
    save_tree(rows, args.output_file)


if __name__ == "__main__":
    main()
