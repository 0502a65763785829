"""KV-tree node type, tree-file reader/writer and synthetic tree generators.

The tree file is the input format of the whole kernel bench: line 1 holds the node
count ``n``; each of the next ``n`` lines holds ``parent id seqlen num_children`` as
space-separated integers.  Node 0 is the root (``parent == -1``) and a parent's id is
always smaller than its children's ids.

Reference: kernel_bench/kv_tree_simple.py:4-10 (node record), :50-64 (reader);
kernel_bench/tree_generation.py:19-94 (level-regular generator and writer).
"""

from __future__ import annotations

import math
import random
from typing import Iterable, List, Sequence


class KVTreeNode:
    """One radix-tree node: ``seqlen`` KV tokens shared by every request below it.

    Mirrors kernel_bench/kv_tree_simple.py:4-10 (same attribute names, same defaults).
    """

    __slots__ = ("parent", "id", "seqlen", "num_children", "requests")

    def __init__(self, parent: int = -1, id: int = -1, seqlen: int = 0, num_children: int = 0):
        self.parent = parent
        self.id = id
        self.seqlen = seqlen
        self.num_children = num_children
        self.requests: List[int] = []

    def __repr__(self) -> str:  # debugging aid only
        return (
            f"KVTreeNode(parent={self.parent}, id={self.id}, seqlen={self.seqlen}, "
            f"num_children={self.num_children}, requests={self.requests})"
        )


def nodes_from_rows(rows: Iterable[Sequence[int]]) -> List[KVTreeNode]:
    """Build node objects from ``[parent, id, seqlen, num_children]`` rows."""
    return [KVTreeNode(int(p), int(i), int(s), int(c)) for p, i, s, c in rows]


def retrive_from_file(filepath: str) -> List[KVTreeNode]:
    """Read a tree file (name kept from kernel_bench/kv_tree_simple.py:50)."""
    with open(filepath, "r") as fh:
        tokens = fh.read().split()
    count = int(tokens[0])
    body = tokens[1 : 1 + 4 * count]
    if len(body) != 4 * count:
        raise ValueError(f"{filepath}: expected {count} node lines")
    return nodes_from_rows(
        (body[4 * k], body[4 * k + 1], body[4 * k + 2], body[4 * k + 3]) for k in range(count)
    )


def generate_tree(layer_sizes: Sequence[int], layer_lengths: Sequence[int]) -> List[List[int]]:
    """Level-regular tree as ``[parent, id, seqlen, num_children]`` rows.

    Ids run level by level; child ``j`` of a level holding ``size`` nodes hangs under
    the previous level's node number ``(j * prev_size) // size``, which spreads the
    children evenly (kernel_bench/tree_generation.py:41-74).
    """
    if len(layer_sizes) != len(layer_lengths):
        raise ValueError("The length of layer_sizes must be equal to the length of layer_lengths.")
    rows: List[List[int]] = []
    prev_first, prev_size = 0, 0
    for depth, (size, seq_len) in enumerate(zip(layer_sizes, layer_lengths)):
        first = len(rows)
        for j in range(size):
            if depth == 0:
                parent = -1
            else:
                parent = prev_first + (j * prev_size) // size
                rows[parent][3] += 1
            rows.append([parent, first + j, seq_len, 0])
        prev_first, prev_size = first, size
    return rows


def generate_irregular_tree(
    seed: int,
    levels: int = 5,
    fanout_range: Sequence[int] = (1, 8),
    len_range: Sequence[int] = (16, 2048),
    max_leaves: int = 1024,
) -> List[List[int]]:
    """Seeded deep irregular tree in the same row format as :func:`generate_tree`.

    Level by level (breadth first) every node of the current level draws a fan-out
    uniformly from ``fanout_range`` (inclusive) and every node draws a context length
    log-uniformly from ``len_range``.  A level stops growing as soon as adding another
    child would push the number of leaves past ``max_leaves``; nodes left without
    children become leaves.  The reference has no generator for such trees (its
    generator is level-regular only, kernel_bench/tree_generation.py:19-76); the file
    format is the reference's.
    """
    rng = random.Random(seed)
    lo, hi = math.log(len_range[0]), math.log(len_range[1])

    def draw_len() -> int:
        return max(len_range[0], min(len_range[1], int(round(math.exp(rng.uniform(lo, hi))))))

    rows: List[List[int]] = [[-1, 0, draw_len(), 0]]
    frontier = [0]
    leaves = 1
    for _ in range(1, levels):
        nxt: List[int] = []
        for parent in frontier:
            fan = rng.randint(fanout_range[0], fanout_range[1])
            for c in range(fan):
                # the first child replaces its parent as a leaf; every further child adds one
                if c > 0 and leaves + 1 > max_leaves:
                    break
                if c > 0:
                    leaves += 1
                nid = len(rows)
                rows.append([parent, nid, draw_len(), 0])
                rows[parent][3] += 1
                nxt.append(nid)
        frontier = nxt
        if not frontier:
            break
    return rows


def save_tree(nodes: Iterable[Sequence[int]], output_path: str) -> None:
    """Write rows in the tree-file format (kernel_bench/tree_generation.py:78-94)."""
    nodes = list(nodes)
    with open(output_path, "w", encoding="utf-8") as fh:
        fh.write(f"{len(nodes)}\n")
        for parent, node_id, seq_len, out_degree in nodes:
            fh.write(f"{parent} {node_id} {seq_len} {out_degree}\n")


def assign_requests(tree_info: List[KVTreeNode]) -> int:
    """Number the leaves 0..B-1 in ascending node id and record each request on every
    node of its root path (kernel_bench/flash_attn_wrap.py:24-33).  Clears any earlier
    assignment first.  Returns the number of requests."""
    for node in tree_info:
        node.requests = []
    count = 0
    for index, node in enumerate(tree_info):
        if node.num_children != 0:
            continue
        walk = index
        while walk != -1:
            tree_info[walk].requests.append(count)
            walk = tree_info[walk].parent
        count += 1
    return count


def kv_prefix_sums(tree_info: List[KVTreeNode]) -> List[int]:
    """``KV_ptrs``: exclusive prefix sums of node lengths, ``n + 1`` entries
    (kernel_bench/flash_attn_wrap.py:13,22)."""
    ptrs = [0]
    for node in tree_info:
        ptrs.append(ptrs[-1] + node.seqlen)
    return ptrs


def root_path(tree_info: List[KVTreeNode], leaf: int) -> List[int]:
    """Node ids from the root down to ``leaf``."""
    chain = []
    walk = leaf
    while walk != -1:
        chain.append(walk)
        walk = tree_info[walk].parent
    chain.reverse()
    return chain
