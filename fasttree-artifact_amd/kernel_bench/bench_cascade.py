"""Multi-level cascade attention, the engine the reference measures with FlashInfer's
``MultiLevelCascadeAttentionWrapper`` (kernel_bench/bench_cascade.py:65-182), on this library's
HIP kernels, with the reference script's command line:

    python bench_cascade.py --node_num_per_level 1,4,8 --node_seqlen_per_level 128,128,128 \
        --num_qo_heads 32 --num_kv_heads 32

A cascade plan names, per tree level, the KV pages of every node of the level and the range of
requests under it (``qo_indptr``); the attention of a request is the merge, over the levels, of
its attention over the one node of each level it lies under.  That is one batched attention per
tree node and a merge per request: every (level, node) becomes one vnode of the tree-decode
kernels -- its KV run the node's pages, its rows the requests under it -- and the second stage
merges a request's rows (``MultiLevelCascadeAttention.plan`` / ``.run``, the wrapper's two calls
with the wrapper's arguments).  The vnodes are arranged as block programs for the device like any
other launch-order plan.  Page size 1 only, as the reference script fixes it.
"""
import argparse
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from fasttree_hip import _lib  # noqa: E402
from fasttree_hip.decode import fasttree_decode  # noqa: E402
from fasttree_hip.planner import place_plan  # noqa: E402


def build_bfs_kv_indices(node_pages_per_level, node_num_per_level, device="cuda"):
    """Page indices of every level's nodes when the tree's pages are numbered in depth-first
    order (the role of kernel_bench/bench_cascade.py:29-62): one int32 tensor per level, the
    nodes of the level back to back."""
    levels = len(node_pages_per_level)
    starts = [np.zeros(n, dtype=np.int64) for n in node_num_per_level]
    cursor = 0
    stack = [(0, 0)]
    while stack:
        level, pos = stack.pop()
        starts[level][pos] = cursor
        cursor += node_pages_per_level[level]
        if level + 1 < levels:
            fan = node_num_per_level[level + 1] // node_num_per_level[level]
            stack.extend((level + 1, pos * fan + i) for i in reversed(range(fan)))
    out = []
    for level in range(levels):
        pages = starts[level][:, None] + np.arange(node_pages_per_level[level])[None, :]
        out.append(torch.from_numpy(pages.reshape(-1).astype(np.int32)).to(device))
    return out


def cascade_lists(qo_indptr_arr, kv_page_indptr_arr, kv_page_indices_arr, kv_last_page_len_arr, page_size, group):
    """The vnode lists of a cascade plan on the host: one vnode per (level, node) that has both
    requests and pages.  Returns ``(kv_entries, (kv_offs, kv_lens, q_offs, q_lens), q_entries,
    (req_entries, req_offs, req_lens), phase_nums, phase_offs, batch_size)`` with the vnodes of
    more than 16 query rows (requests x group) first, as the decode kernels take them."""
    if page_size != 1:
        raise ValueError("page_size must be 1 (one token per pool slot), as in the reference script")
    host = lambda t: np.asarray(t.cpu() if hasattr(t, "cpu") else t, dtype=np.int64).reshape(-1)
    vnodes = []                                   # (rows, kv_off, kv_len, first request, requests)
    kv_entries = []
    batch = 0
    for qo, kv_ptr, pages, last in zip(qo_indptr_arr, kv_page_indptr_arr, kv_page_indices_arr, kv_last_page_len_arr):
        qo, kv_ptr, pages, last = host(qo), host(kv_ptr), host(pages), host(last)
        if len(qo) != len(kv_ptr) or len(last) != len(qo) - 1:
            raise ValueError("qo_indptr, kv_page_indptr and kv_last_page_len of a level disagree on its number of nodes")
        batch = max(batch, int(qo[-1]))
        for node in range(len(qo) - 1):
            first, count = int(qo[node]), int(qo[node + 1] - qo[node])
            tokens = pages[kv_ptr[node]: kv_ptr[node + 1]]
            if len(tokens) and last[node] != 1:
                raise ValueError("kv_last_page_len must be 1 with page_size 1")
            if count <= 0 or len(tokens) == 0:
                continue
            vnodes.append((count * group, len(kv_entries), len(tokens), first, count))
            kv_entries.extend(tokens.tolist())
    wide = [v for v in vnodes if v[0] > 16]
    narrow = [v for v in vnodes if v[0] <= 16]
    kv_offs, kv_lens, q_offs, q_lens, q_entries = [], [], [], [], []
    for _, off, length, first, count in wide + narrow:
        kv_offs.append(off)
        kv_lens.append(length)
        q_offs.append(len(q_entries))
        q_lens.append(count)
        q_entries.extend(range(first, first + count))
    rows_of = [[] for _ in range(batch)]
    for row, request in enumerate(q_entries):
        rows_of[request].append(row)
    req_lens = [len(r) for r in rows_of]
    req_offs = np.concatenate([[0], np.cumsum(req_lens)[:-1]]).astype(np.int64) if batch else np.zeros(0, dtype=np.int64)
    req_entries = [row for rows in rows_of for row in rows]
    i32 = lambda x: np.asarray(x, dtype=np.int32).reshape(-1)
    return (i32(kv_entries), (i32(kv_offs), i32(kv_lens), i32(q_offs), i32(q_lens)), i32(q_entries),
            (i32(req_entries), i32(req_offs), i32(req_lens)), [len(wide), len(narrow)], [0, len(wide)], batch)


class MultiLevelCascadeAttention:
    """``plan`` and ``run`` with the arguments the reference gives FlashInfer's wrapper
    (kernel_bench/bench_cascade.py:112,151-160,172).  ``workspace_buffer`` is accepted for the
    signature; the partial results live in buffers that ``plan`` allocates."""

    def __init__(self, num_levels, workspace_buffer=None, kv_layout="NHD"):
        if kv_layout != "NHD":
            raise ValueError("kv_layout must be NHD: [pages, 2, page_size, kv heads, head_dim]")
        self.num_levels = int(num_levels)
        self._aux = None

    def plan(self, qo_indptr_arr, kv_page_indptr_arr, kv_page_indices_arr, kv_last_page_len_arr,
             num_qo_heads, num_kv_heads, head_dim, page_size, *, device="cuda", sm_scale=None):
        if not (len(qo_indptr_arr) == len(kv_page_indptr_arr) == len(kv_page_indices_arr)
                == len(kv_last_page_len_arr) == self.num_levels):
            raise ValueError(f"expected the arrays of {self.num_levels} levels")
        if num_qo_heads % num_kv_heads:
            raise ValueError("num_qo_heads must be a multiple of num_kv_heads")
        group = num_qo_heads // num_kv_heads
        kv_entries, vnodes, q_entries, per_request, nums, offs, batch = cascade_lists(
            qo_indptr_arr, kv_page_indptr_arr, kv_page_indices_arr, kv_last_page_len_arr, page_size, group)
        self.batch_size, self.heads, self.head_dim = batch, (num_qo_heads, num_kv_heads), head_dim
        self.sm_scale = float(sm_scale) if sm_scale is not None else 1.0 / (head_dim ** 0.5)
        self._aux = place_plan(kv_entries, vnodes, q_entries, per_request, nums, offs, batch, num_qo_heads, num_kv_heads,
                               head_dim, device=device, launch_order=True)
        # (tile arguments of the decode call: any vnode of more than 16 rows is a wide one)
        self._tiles = ([128 // group + 1, max(1, 16 // group)], [32, 32])

    def run(self, q, paged_kv_cache, out=None):
        if self._aux is None:
            raise RuntimeError("plan() has not been called")
        if paged_kv_cache.dim() != 5 or paged_kv_cache.shape[1] != 2 or paged_kv_cache.shape[2] != 1:
            raise _lib.FastTreeLibraryError("paged_kv_cache must be [pages, 2, 1, kv heads, head_dim]")
        k, v = paged_kv_cache[:, 0, 0], paged_kv_cache[:, 1, 0]        # [pages, Hkv, D] views: a page is a pool slot
        o = torch.empty_like(q) if out is None else out
        fasttree_decode(q, k, v, o, *self._aux, self._tiles[0], self._tiles[1], self.sm_scale)
        return o


def main(argv=None):
    parser = argparse.ArgumentParser(description="multi-level cascade attention on the tree-decode kernels")
    parser.add_argument("--node_num_per_level", type=str, default="1,4,8")
    parser.add_argument("--node_seqlen_per_level", type=str, default="128,128,128")
    parser.add_argument("--num_qo_heads", type=int, default=32)
    parser.add_argument("--num_kv_heads", type=int, default=32)
    args = parser.parse_args(argv)

    node_num_per_level = list(map(int, args.node_num_per_level.split(",")))
    node_seqlen_per_level = list(map(int, args.node_seqlen_per_level.split(",")))
    head_dim, page_size = 128, 1                       # (kernel_bench/bench_cascade.py:101-103)
    total_pages = sum(n * s for n, s in zip(node_num_per_level, node_seqlen_per_level))
    batch_size = node_num_per_level[-1]

    wrapper = MultiLevelCascadeAttention(len(node_num_per_level), None, "NHD")
    kv_page_indices_arr = build_bfs_kv_indices(node_seqlen_per_level, node_num_per_level)
    kv_page_indptr_arr = [torch.arange(n + 1, device="cuda", dtype=torch.int32) * s
                          for n, s in zip(node_num_per_level, node_seqlen_per_level)]
    kv_last_page_len_arr = [torch.full((n,), page_size, dtype=torch.int32, device="cuda") for n in node_num_per_level]
    qo_indptr_arr = [torch.linspace(0, batch_size, n + 1, dtype=torch.int32, device="cuda") for n in node_num_per_level]
    kv_cache = torch.randn(total_pages, 2, page_size, args.num_kv_heads, head_dim, dtype=torch.float16, device="cuda")
    q = torch.randn(batch_size, args.num_qo_heads, head_dim, dtype=torch.float16, device="cuda")
    wrapper.plan(qo_indptr_arr, kv_page_indptr_arr, kv_page_indices_arr, kv_last_page_len_arr,
                 args.num_qo_heads, args.num_kv_heads, head_dim, page_size)

    from benchmark import QUANTILES, do_bench
    out = wrapper.run(q, kv_cache)
    t, _, _ = do_bench(lambda: wrapper.run(q, kv_cache, out=out), quantiles=QUANTILES)
    # (the label is the one the reference's parse_output.py looks for, kernel_bench/parse_output.py:118;
    # the engine behind it here is this library, not FlashInfer)
    print("FlashInfer MutliLevelCascadeAttn time:", t)
    return {"cascade": t, "out": out, "q": q, "kv_cache": kv_cache, "plan": (qo_indptr_arr, kv_page_indptr_arr, kv_page_indices_arr)}


if __name__ == "__main__":
    main()
