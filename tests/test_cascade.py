"""Multi-level cascade attention on the tree-decode kernels (kernel_bench/bench_cascade.py here; the
engine the reference measures through FlashInfer's wrapper, kernel_bench/bench_cascade.py:65-182 of
the reference): the page numbering and the vnode lists of a plan on the CPU, worked by hand, and
-- on the GPU -- ``plan`` / ``run`` against the fp64 dense oracle over every request's root path."""
import math
import os
import sys

import numpy as np
import pytest
import torch

import fasttree_oracle as oracle
from helpers import assert_parity

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fasttree-artifact_amd", "kernel_bench"))
import bench_cascade  # noqa: E402


def _plan_arrays(nodes, lens, device="cpu"):
    batch = nodes[-1]
    pages = bench_cascade.build_bfs_kv_indices(lens, nodes, device=device)
    indptr = [torch.arange(n + 1, dtype=torch.int32, device=device) * s for n, s in zip(nodes, lens)]
    last = [torch.full((n,), 1, dtype=torch.int32, device=device) for n in nodes]
    qo = [torch.linspace(0, batch, n + 1, dtype=torch.int32, device=device) for n in nodes]
    return qo, indptr, pages, last


def test_pages_are_numbered_depth_first():
    """1 root of 3 pages, 2 children of 2, 4 leaves of 1 (kernel_bench/bench_cascade.py:29-62 by hand):
    root 0-2; child 0 3-4, its leaves 5 and 6; child 1 7-8, its leaves 9 and 10."""
    pages = bench_cascade.build_bfs_kv_indices([3, 2, 1], [1, 2, 4], device="cpu")
    assert [p.tolist() for p in pages] == [[0, 1, 2], [3, 4, 7, 8], [5, 6, 9, 10]]
    assert all(p.dtype == torch.int32 for p in pages)


def test_cascade_lists_by_hand():
    """The same tree, 4 requests, 8 query heads per kv head: root and children have more than 16
    rows (32 and 16+... = 2 requests x 8 = 16 rows: narrow), leaves 8 rows."""
    qo, indptr, pages, last = _plan_arrays([1, 2, 4], [3, 2, 1])
    kv_entries, vnodes, q_entries, per_request, nums, offs, batch = bench_cascade.cascade_lists(qo, indptr, pages, last, 1, 8)
    assert batch == 4 and nums == [1, 6] and offs == [0, 1]
    assert kv_entries.tolist() == [0, 1, 2, 3, 4, 7, 8, 5, 6, 9, 10]
    kv_offs, kv_lens, q_offs, q_lens = (x.tolist() for x in vnodes)
    assert kv_offs == [0, 3, 5, 7, 8, 9, 10] and kv_lens == [3, 2, 2, 1, 1, 1, 1]
    assert q_lens == [4, 2, 2, 1, 1, 1, 1] and q_offs == [0, 4, 6, 8, 9, 10, 11]
    assert q_entries.tolist() == [0, 1, 2, 3, 0, 1, 2, 3, 0, 1, 2, 3]
    entries, req_offs, req_lens = (x.tolist() for x in per_request)
    assert req_lens == [3, 3, 3, 3] and req_offs == [0, 3, 6, 9] and entries == [0, 4, 8, 1, 5, 9, 2, 6, 10, 3, 7, 11]
    # with one query head per kv head nothing has more than 16 rows
    assert bench_cascade.cascade_lists(qo, indptr, pages, last, 1, 1)[4] == [0, 7]
    with pytest.raises(ValueError):
        bench_cascade.cascade_lists(qo, indptr, pages, last, 16, 8)
    with pytest.raises(ValueError):
        bench_cascade.MultiLevelCascadeAttention(3, None, "HND")


@pytest.mark.gpu
@pytest.mark.parametrize("nodes,lens,heads", [
    ([1, 4, 8], [128, 128, 128], (32, 32)),       # the reference script's defaults
    ([1, 10, 400], [4000, 400, 40], (32, 8)),     # the headline tree
    ([1, 2, 64], [8, 256, 32], (16, 1)),
    ([1, 5, 20, 60], [77, 1, 130, 33], (32, 4)),
])
def test_cascade_matches_dense_attention(nodes, lens, heads, device):
    print("\n[gpu case] cascade", nodes, lens, heads, flush=True)
    hq, hkv = heads
    d = 128
    qo, indptr, pages, last = _plan_arrays(nodes, lens, device=device)
    total = sum(n * s for n, s in zip(nodes, lens))
    gen = torch.Generator(device="cpu").manual_seed(7)
    kv_cache = torch.randn(total, 2, 1, hkv, d, generator=gen, dtype=torch.float32).to(torch.float16).to(device)
    q = torch.randn(nodes[-1], hq, d, generator=gen, dtype=torch.float32).to(torch.float16).to(device)
    wrapper = bench_cascade.MultiLevelCascadeAttention(len(nodes), None, "NHD")
    wrapper.plan(qo, indptr, pages, last, hq, hkv, d, 1, device=device)
    o = wrapper.run(q, kv_cache)
    again = wrapper.run(q, kv_cache, out=torch.empty_like(o))
    torch.cuda.synchronize()
    assert torch.equal(o, again)
    # a request's path: the pages of the node it lies under, level by level
    batch = nodes[-1]
    host_pages = [p.cpu().numpy() for p in pages]
    paths = []
    for r in range(batch):
        tokens = []
        for level, (n, s) in enumerate(zip(nodes, lens)):
            node = r * n // batch
            tokens.append(host_pages[level][node * s:(node + 1) * s])
        paths.append(np.concatenate(tokens))
    sample = list(range(0, batch, max(1, batch // 24)))
    k_pool, v_pool = kv_cache[:, 0, 0].cpu(), kv_cache[:, 1, 0].cpu()
    want = oracle.dense_attention(q[sample].cpu(), k_pool, v_pool, [paths[r] for r in sample], 1.0 / math.sqrt(d))
    assert_parity(o[sample], want.to(torch.float16), f"cascade {nodes} {lens} {heads}")
