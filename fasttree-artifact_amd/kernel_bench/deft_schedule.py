"""DeFT's schedule of a tree decode, run through this library's kernels.

The reference benchmarks DeFT-Flatten with a Triton kernel of its own (kernel_bench/DeFT.py):
the tree's tokens are laid out in depth-first order and cut into *subtrees* of ``subtree_len``
tokens (kernel_bench/DeFT.py:14-55; 128 in kernel_bench/benchmark.py:183); one thread block per
(subtree, head) attends the pieces of nodes that fall into its subtree, for all queries under
those nodes, masking per query the pieces that are not on its path (DeFT.py:76-135, 195-340),
and a second kernel merges the partial results of every query (DeFT.py:410-507).

Here the same partition becomes a launch of block programs: one program per subtree, whose
vnodes are the subtree's node pieces -- a piece is attended by exactly the requests under its
node, so the bit mask of the Triton kernel turns into one vnode per piece (cut further into row
chunks of what one block serves per pass) -- and the library's second stage merges per request.
What is compared is the schedule: equal *token* counts per block whatever the number of queries
that share them, no cost model, no merging of nodes into their children.
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from fasttree_hip.launch_schedule import BLOCK_ROWS, LaunchPhases  # noqa: E402


def group_subtrees(tree_info, subtree_len):
    """The depth-first partition of kernel_bench/DeFT.py:29-55 without recursion: a list of
    subtrees, each a list of (node, first token, end token) pieces of ``subtree_len`` tokens in
    total (the last one maybe fewer)."""
    children = [[] for _ in tree_info]
    for index, node in enumerate(tree_info):
        if node.parent >= 0:
            children[node.parent].append(index)
    subtrees, current, filled = [], [], 0
    stack = [0] if tree_info else []
    while stack:
        node = stack.pop()
        pos, length = 0, tree_info[node].seqlen
        while filled + length - pos >= subtree_len:      # the piece that fills the subtree
            take = subtree_len - filled
            current.append((node, pos, pos + take))
            subtrees.append(current)
            current, filled, pos = [], 0, pos + take
        # the rest of the node opens (or continues) the next subtree; a node that ends exactly
        # where a subtree does leaves nothing (DeFT.py:40-44 goes on to its children), nor does a
        # node without tokens: empty pieces are dropped below
        current.append((node, pos, length))
        filled += length - pos
        stack.extend(reversed(children[node]))           # children in ascending id, depth first
    if current:
        subtrees.append(current)
    return [[p for p in sub if p[2] > p[1]] for sub in subtrees if any(p[2] > p[1] for p in sub)]


def deft_lists(tree_info, KV_ptrs, batch_size, group, subtree_len=128, block_rows=BLOCK_ROWS):
    """The vnode lists, per-request lists and program table of the DeFT schedule (numpy)."""
    cap = max(1, int(block_rows) // max(1, int(group)))          # requests per vnode
    kv_offs, kv_lens, q_offs, q_lens, rows, table = [], [], [], [], [], []
    row = 0
    for pieces in group_subtrees(tree_info, subtree_len):
        first = len(kv_offs)
        for node, start, end in pieces:
            requests = sorted(tree_info[node].requests)
            for lo in range(0, len(requests), cap):
                part = requests[lo: lo + cap]
                kv_offs.append(int(KV_ptrs[node]) + start)
                kv_lens.append(end - start)
                q_offs.append(row)
                q_lens.append(len(part))
                rows.append(part)
                row += len(part)
        if len(kv_offs) > first:
            table.append((first, len(kv_offs), 0, 0))
    q_entries = np.concatenate([np.asarray(r, dtype=np.int64) for r in rows]) if rows else np.zeros(0, dtype=np.int64)
    # scratch rows of every request, in row order, then the reference's padding (kernel_bench/fasttree.py:233-262)
    by_req = np.argsort(q_entries, kind="stable")
    req_lens = np.bincount(q_entries, minlength=int(batch_size))[: int(batch_size)]
    req_offs = np.concatenate([[0], np.cumsum(req_lens)[:-1]]) if batch_size else np.zeros(0, dtype=np.int64)
    req_entries = np.concatenate([by_req, np.full(32, -1, dtype=np.int64)])
    i32 = lambda x: np.asarray(x, dtype=np.int32)
    return dict(kv_offs=i32(kv_offs), kv_lens=i32(kv_lens), q_offs=i32(q_offs), q_lens=i32(q_lens), q_entries=i32(q_entries),
                req_entries=i32(req_entries), req_offs=i32(req_offs), req_lens=i32(req_lens),
                prog_table=i32(table).reshape(-1, 4))


def deft_preparation(tree_info, KV_ptrs, batch_size, num_qo_heads, num_kv_heads, head_dim, subtree_len=128, device="cuda",
                     kv_slot_map=None):
    """The thirteen arguments ``fasttree_decode`` takes after Q, K, V and the output (the tuple
    ``fasttree_preparation`` returns), for the DeFT schedule.  Token t of the flattened tree
    lies in pool slot ``kv_slot_map[t]`` (default: slot t, as ``qkv_preparation`` lays the pool out)."""
    import torch

    lists = deft_lists(tree_info, KV_ptrs, batch_size, max(1, num_qo_heads // num_kv_heads), subtree_len)
    to_device = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(device)
    slots = np.arange(int(KV_ptrs[-1]), dtype=np.int64)
    if kv_slot_map is not None:
        slots = np.asarray(kv_slot_map, dtype=np.int64)[slots]
    kv_entries = np.concatenate([slots, np.full(32, -1, dtype=np.int64)]).astype(np.int32)
    rows = int(lists["q_entries"].shape[0])
    phases = LaunchPhases([int(lists["kv_offs"].shape[0]), 0])
    phases.prog_table = to_device(lists["prog_table"].reshape(-1))
    phases.num_programs = int(lists["prog_table"].shape[0])
    phases.narrow_in_programs = 0
    mid_o = torch.empty((rows, num_qo_heads, head_dim), dtype=torch.float32, device=device)
    mid_lse = torch.empty((rows, num_qo_heads), dtype=torch.float32, device=device)
    return (to_device(kv_entries), to_device(lists["kv_offs"]), to_device(lists["kv_lens"]), to_device(lists["q_entries"]),
            to_device(lists["q_offs"]), to_device(lists["q_lens"]), to_device(lists["req_entries"]),
            to_device(lists["req_offs"]), to_device(lists["req_lens"]), mid_o, mid_lse, phases, [0, phases[0]])
