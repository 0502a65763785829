"""DeFT-Flatten, the tree-attention engine the reference's benchmark compares FastTree with
(kernel_bench/DeFT.py), on this library's HIP kernels: ``DeFT_preparation`` and ``DeFT_decode``
with the reference's signatures (DeFT.py:58-64, 489-512; called at kernel_bench/benchmark.py:
180-211).

The tree's tokens are taken in depth-first order and cut into subtrees of ``subtree_len``
tokens; a subtree is a list of node pieces.  Its query set is every request under any of its
pieces; per group of ``mask_len`` requests of that set and per token, one 64-bit word holds the
requests of the group that attend the token.  One thread block per (subtree, KV head) computes the
partial attention of the whole query set over the subtree's tokens with those masks
(``ft_deft_stage1``), a second launch merges each request's partial rows (``ft_stage2``, the same
arithmetic as DeFT.py:406-486).

As in the reference, the KV index entries address the per-request gathered cache
``K_cache.view(-1, Hkv, D)``: a token of a node is read from the copy of the node's first request
(DeFT.py:88-91).  With ``KV_ptrs`` (and optionally ``kv_slot_map``) given, they address the tree
pool of ``qkv_preparation`` instead, which the reference's version cannot.
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from fasttree_hip import _lib  # noqa: E402


def _children_of(tree_info):
    children = [[] for _ in tree_info]
    for index, node in enumerate(tree_info):
        if node.parent >= 0:
            children[node.parent].append(index)
    return children


def group_subtree(tree_info, subtree_len):
    """The partition of DeFT.py:29-55, without recursion: a list of subtrees, each a list of
    ``(node, start, end)`` pieces in depth-first order (children in ascending id).  A piece that
    fills its subtree closes it; what is left of the node opens the next one.  A node without
    tokens still contributes an empty piece (its requests join the query set, DeFT.py:50-52)."""
    children = _children_of(tree_info)
    subtrees, filled = [[]], 0
    stack = [0] if len(tree_info) else []
    while stack:
        node = stack.pop()
        pos, length = 0, tree_info[node].seqlen
        while filled + length - pos >= subtree_len:
            take = subtree_len - filled
            subtrees[-1].append((node, pos, pos + take))
            subtrees.append([])
            pos, filled = pos + take, 0
            if pos == length:
                break
        else:
            subtrees[-1].append((node, pos, length))
            filled += length - pos
        stack.extend(reversed(children[node]))
    if not subtrees[-1]:
        subtrees.pop()
    return subtrees


def deft_lists(tree_info, batch_size, max_seqlen, subtree_len, mask_len, KV_ptrs=None, kv_slot_map=None):
    """The eleven index arrays of DeFT.py:73-154 as numpy arrays (int32, the masks int64)."""
    total = sum(node.seqlen for node in tree_info)
    subtrees = group_subtree(tree_info, subtree_len)
    if len(subtrees) != (total - 1) // subtree_len + 1:
        raise AssertionError("Group subtree error!")                 # DeFT.py:71-72
    prefix = [0] * len(tree_info)                                    # tokens above a node on its root path
    for index, node in enumerate(tree_info):
        if node.parent >= 0:
            prefix[index] = prefix[node.parent] + tree_info[node.parent].seqlen
    kv_entries, kv_offs, kv_lens, q_entries, q_offs, q_lens, masks, mask_offs = [], [], [], [], [], [], [], []
    for pieces in subtrees:
        kv_offs.append(len(kv_entries))
        q_offs.append(len(q_entries))
        mask_offs.append(len(masks))
        for node, start, end in pieces:
            if KV_ptrs is None:
                first = prefix[node] + start + tree_info[node].requests[0] * max_seqlen
            else:
                first = int(KV_ptrs[node]) + start
            kv_entries.extend(range(first, first + end - start))
        members = sorted({r for node, _, _ in pieces for r in tree_info[node].requests})
        q_entries.extend(members)
        position = {r: i for i, r in enumerate(members)}
        for group in range((len(members) - 1) // mask_len + 1):
            lo, hi = group * mask_len, min(len(members), (group + 1) * mask_len)
            for node, start, end in pieces:
                word = 0
                for r in tree_info[node].requests:
                    if lo <= position[r] < hi:
                        word |= 1 << (position[r] - lo)
                if word >= 1 << 63:
                    word -= 1 << 64                                    # (as a signed 64-bit value, DeFT.py:108-109)
                masks.extend([word] * (end - start))
        kv_lens.append(len(kv_entries) - kv_offs[-1])
        q_lens.append(len(members))
    req_rows = [[] for _ in range(batch_size)]
    for row, request in enumerate(q_entries):
        req_rows[request].append(row)
    req_lens = [len(rows) for rows in req_rows]
    req_offs = np.concatenate([[0], np.cumsum(req_lens)[:-1]]) if batch_size else []
    if kv_slot_map is not None and KV_ptrs is not None:
        kv_entries = np.asarray(kv_slot_map, dtype=np.int64)[np.asarray(kv_entries, dtype=np.int64)].tolist()
    i32 = lambda x: np.asarray(x, dtype=np.int32).reshape(-1)
    return (i32(list(kv_entries) + [-1] * 32), i32(kv_offs), i32(kv_lens), i32(q_entries), i32(q_offs), i32(q_lens),
            np.asarray(masks, dtype=np.int64).reshape(-1), i32(mask_offs),
            i32([row for rows in req_rows for row in rows] + [-1] * 32), i32(req_offs), i32(req_lens))


def DeFT_preparation(Tree_info, K_cache, subtree_len, mask_len, num_qo_heads, head_dim, *, device="cuda",
                     KV_ptrs=None, kv_slot_map=None):
    """Drop-in for kernel_bench/DeFT.py:58-191: the thirteen arguments ``DeFT_decode`` takes after
    the output tensor.  ``K_cache`` is only asked for its batch size and padded length."""
    batch_size, max_seqlen = int(K_cache.shape[0]), int(K_cache.shape[1])
    lists = deft_lists(Tree_info, batch_size, max_seqlen, subtree_len, mask_len, KV_ptrs, kv_slot_map)
    put = lambda arr: torch.from_numpy(np.ascontiguousarray(arr)).to(device)
    rows = int(lists[3].shape[0])
    mid_o = torch.empty((rows, num_qo_heads, head_dim), dtype=torch.float32, device=device)
    mid_lse = torch.empty((rows, num_qo_heads), dtype=torch.float32, device=device)
    return tuple(put(x) for x in lists) + (mid_o, mid_lse)


def DeFT_decode(q, k_buffer, v_buffer, o, vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens,
                vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, causalmask, causalmask_offset,
                req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens, mid_o, mid_lse,
                Q_TILE_SIZE, KV_TILE_SIZE, sm_scale, mask_len, logit_cap=-1):
    """Drop-in for kernel_bench/DeFT.py:489-560.  ``Q_TILE_SIZE`` and ``KV_TILE_SIZE`` are accepted
    for the signature: a block serves 128 query rows per pass and 32 tokens per step whatever they
    say.  ``logit_cap`` is ignored, as in the reference."""
    assert q.shape[-1] == k_buffer.shape[-1]
    for t in (q, k_buffer, v_buffer, o, mid_o, mid_lse, vnode_to_kv_entries, causalmask):
        if not t.is_cuda:
            raise _lib.FastTreeLibraryError("DeFT_decode needs device tensors; there is no CPU path")
    if causalmask.dtype != torch.int64 or not causalmask.is_contiguous():
        raise _lib.FastTreeLibraryError("causalmask must be a contiguous int64 tensor")
    for t in (vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens, vnode_to_q_entries, vnode_to_q_offs,
              vnode_to_q_lens, causalmask_offset, req_to_vnode_entries, req_to_vnode_offs, req_to_vnode_lens):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise _lib.FastTreeLibraryError("index tensors must be contiguous int32")
    dtype = {torch.float16: _lib.FT_DTYPE_F16, torch.bfloat16: _lib.FT_DTYPE_BF16}.get(q.dtype)
    if dtype is None or k_buffer.dtype != q.dtype or v_buffer.dtype != q.dtype or o.dtype != q.dtype:
        raise _lib.FastTreeLibraryError("q, k, v and o must share one dtype, fp16 or bf16")
    rc = _lib.load().ft_deft_decode(
        q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), o.data_ptr(),
        q.stride(0), q.stride(1), k_buffer.stride(0), k_buffer.stride(1), v_buffer.stride(0), v_buffer.stride(1),
        o.stride(0), o.stride(1),
        vnode_to_kv_entries.data_ptr(), vnode_to_kv_offs.data_ptr(), vnode_to_kv_lens.data_ptr(),
        vnode_to_q_entries.data_ptr(), vnode_to_q_offs.data_ptr(), vnode_to_q_lens.data_ptr(),
        causalmask.data_ptr(), causalmask_offset.data_ptr(),
        req_to_vnode_entries.data_ptr(), req_to_vnode_offs.data_ptr(), req_to_vnode_lens.data_ptr(),
        mid_o.data_ptr(), mid_o.stride(0), mid_o.stride(1), mid_lse.data_ptr(), mid_lse.stride(0),
        int(vnode_to_q_offs.shape[0]), q.shape[0], q.shape[1], k_buffer.shape[1], q.shape[-1],
        int(mask_len), float(sm_scale), dtype, torch.cuda.current_stream(q.device).cuda_stream)
    _lib.check(rc, "ft_deft_decode")
