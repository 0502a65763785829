"""CPU oracle for the FastTree decode path.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU, what the reference computes on this path, so that the
HIP kernels and the host planner can be checked against it.  Only the tests, the smoke
check and the bench's ``cpu_baseline`` leg may import it; the product never does and has
no CPU fallback.

Contents and the reference lines each part follows (paths relative to the reference
checkout):

* ``dense_attention``            per-request soft-max attention over the request's root
                                 path in fp64 -- the identity the whole tree scheme must
                                 satisfy (comparison baseline of kernel_bench/benchmark.py:216-220).
* ``stage1_arith``               the arithmetic of _fwd_fasttree_decode_stage1,
                                 kernel_bench/fasttree.py:328-413: KV tiles of KV_TILE keys,
                                 fp32 scores, scale, -1e6 mask, online soft-max with natural
                                 exp, probabilities rounded to the storage type before P.V,
                                 fp32 accumulation, partial normalised by its own sum,
                                 lse = log(sum) + max.
* ``stage2_arith``               _fwd_fasttree_decoding_stage2, fasttree.py:498-546: tiles of
                                 4 partials, running max / sum, missing entries count as
                                 lse = -inf, o = 0; result rounded to the output type.
* ``decode_arith_for_requests``  both of the above for a few requests of a given plan (every
                                 scratch row of a sampled request as a one-request vnode over
                                 the same KV slice): the like-for-like reference of the
                                 bfloat16 cases, where the storage type is coarser than the
                                 parity bar.
* ``plan``                       cost model, greedy splitter, 3-pass adaptation and vnode
                                 emission, fasttree.py:30-96 and :111-262.
* ``gathered_attention_torch``   the "no prefix sharing" formulation on the CPU with PyTorch
                                 ops: every request attends over its own gathered copy of the
                                 path KV (layout of kernel_bench/flash_attn_wrap.py:36-67);
                                 this is what the bench times as the CPU baseline.

How the oracle itself is pinned (tests/test_oracle.py): ``plan`` against 207 planner
fixtures written by the reference planner (tests/golden/planner_goldens.json), plus the
hand-derived known answers; ``stage1_arith``/``stage2_arith`` and ``dense_attention``
against outputs of the reference's own kernels executed under Triton's CPU interpreter
(tests/golden/kernel_*.npz), plus closed forms (single key, uniform keys, split
invariance); ``decode_arith_for_requests`` against the same kernel outputs for the requests it
is given and against the whole-plan arithmetic.  No function here is left unpinned.
"""

from __future__ import annotations

import math
from collections import deque
from typing import List, Sequence

import numpy as np
import torch

MASK_VALUE = -1.0e6  # kernel_bench/fasttree.py:377


# ----------------------------------------------------------------------------------------
# numerics
# ----------------------------------------------------------------------------------------

def dense_attention(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                    path_tokens: Sequence[np.ndarray], sm_scale: float) -> torch.Tensor:
    """fp64 ``softmax(scale * q K^T) V`` per request; query head h reads KV head h // g."""
    batch, hq, d = q.shape
    hkv = k_pool.shape[1]
    g = hq // hkv
    out = torch.empty((batch, hq, d), dtype=torch.float64)
    for r in range(batch):
        idx = torch.as_tensor(np.asarray(path_tokens[r]), dtype=torch.long)
        k = k_pool[idx].to(torch.float64)            # [L, Hkv, D]
        v = v_pool[idx].to(torch.float64)
        qr = q[r].to(torch.float64).view(hkv, g, d)  # head h = kv * g + j
        scores = torch.einsum("kgd,lkd->kgl", qr, k) * sm_scale
        prob = torch.softmax(scores, dim=-1)
        out[r] = torch.einsum("kgl,lkd->kgd", prob, v).reshape(hq, d)
    return out


def stage1_arith(q, k_pool, v_pool, kv_entries, kv_offs, kv_lens, q_entries, q_offs, q_lens,
                 kv_tile: int, sm_scale: float, rows: int):
    """Partial attention per vnode with the reference kernel's rounding points.
    Returns ``mid_o [rows, Hq, D]`` and ``mid_lse [rows, Hq]`` in fp32."""
    hq, d = q.shape[1], q.shape[2]
    hkv = k_pool.shape[1]
    g = hq // hkv
    store = q.dtype
    mid_o = torch.zeros((rows, hq, d), dtype=torch.float32)
    mid_lse = torch.zeros((rows, hq), dtype=torch.float32)
    kv_entries = np.asarray(kv_entries)
    for vn in range(len(kv_offs)):
        reqs = np.asarray(q_entries[q_offs[vn]: q_offs[vn] + q_lens[vn]])
        slots = torch.as_tensor(kv_entries[kv_offs[vn]: kv_offs[vn] + kv_lens[vn]].astype(np.int64))
        qv = q[torch.as_tensor(reqs, dtype=torch.long)].to(torch.float32)      # [n, Hq, D]
        n = qv.shape[0]
        acc = torch.zeros((n, hq, d), dtype=torch.float32)
        total = torch.zeros((n, hq), dtype=torch.float32)
        peak = torch.full((n, hq), float("-inf"), dtype=torch.float32)
        for lo in range(0, len(slots), kv_tile):
            part = slots[lo: lo + kv_tile]
            k = k_pool[part].to(torch.float32).repeat_interleave(g, dim=1)     # [t, Hq, D]
            v = v_pool[part].to(torch.float32).repeat_interleave(g, dim=1)
            s = torch.einsum("nhd,thd->nht", qv, k) * np.float32(sm_scale)
            pad = kv_tile - len(part)
            if pad:  # masked tail of the tile
                s = torch.cat([s, torch.full((n, hq, pad), MASK_VALUE, dtype=torch.float32)], dim=-1)
                v = torch.cat([v, torch.zeros((pad, hq, d), dtype=torch.float32)], dim=0)
            new_peak = torch.maximum(s.max(dim=-1).values, peak)
            e = torch.exp(s - new_peak[..., None])
            shrink = torch.exp(peak - new_peak)
            total = total * shrink + e.sum(dim=-1)
            acc = acc * shrink[..., None] + torch.einsum("nht,thd->nhd", e.to(store).to(torch.float32), v)
            peak = new_peak
        rows_here = slice(q_offs[vn], q_offs[vn] + n)
        mid_o[rows_here] = acc / total[..., None]
        mid_lse[rows_here] = torch.log(total) + peak
    return mid_o, mid_lse


def stage2_arith(req_entries, req_offs, req_lens, mid_o, mid_lse, out_dtype, node_tile: int = 4):
    """Merge of each request's partial rows, 4 at a time, as the reference kernel does."""
    batch = len(req_offs)
    hq, d = mid_o.shape[1], mid_o.shape[2]
    out = torch.empty((batch, hq, d), dtype=out_dtype)
    for r in range(batch):
        rows = list(req_entries[req_offs[r]: req_offs[r] + req_lens[r]])
        total = torch.zeros((hq,), dtype=torch.float32)
        peak = torch.full((hq,), float("-inf"), dtype=torch.float32)
        acc = torch.zeros((hq, d), dtype=torch.float32)
        for lo in range(0, len(rows), node_tile):
            idx = torch.as_tensor(rows[lo: lo + node_tile], dtype=torch.long)
            lse = mid_lse[idx]                                   # [t, Hq]
            part = mid_o[idx]                                    # [t, Hq, D]
            new_peak = torch.maximum(lse.max(dim=0).values, peak)
            w = torch.exp(lse - new_peak)
            keep = torch.exp(peak - new_peak)
            total = total * keep + w.sum(dim=0)
            acc = acc * keep[:, None] + (w[..., None] * part).sum(dim=0)
            peak = new_peak
        out[r] = (acc / total[:, None]).to(out_dtype)
    return out


def fasttree_decode_arith(q, k_pool, v_pool, plan, kv_tile: int, sm_scale: float):
    """Both stages over a plan object with the planner's list attributes; returns
    ``(o, mid_o, mid_lse)``."""
    n_pad = 32
    mid_o, mid_lse = stage1_arith(
        q, k_pool, v_pool, np.asarray(plan.vnode_to_kv_entries)[:-n_pad], plan.vnode_to_kv_offs,
        plan.vnode_to_kv_lens, plan.vnode_to_q_entries, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
        kv_tile, sm_scale, len(plan.vnode_to_q_entries))
    o = stage2_arith(plan.req_to_vnode_entries[:-n_pad], plan.req_to_vnode_offs, plan.req_to_vnode_lens,
                     mid_o, mid_lse, q.dtype)
    return o, mid_o, mid_lse


def decode_arith_for_requests(q, k_pool, v_pool, lists, sample, kv_tile: int, sm_scale: float, remap=None):
    """The two-stage arithmetic (stage1_arith, stage2_arith: P rounded to the storage type before
    P.V, fp32 accumulation, the output rounded to the storage type; kernel_bench/fasttree.py:
    384-413, 534-546) for the requests ``sample`` only, on a given plan: ``lists`` are the nine
    index arrays of kernel_bench/fasttree.py:265-280 as numpy arrays (any vnode order).  Every
    scratch row of a sampled request becomes a one-request vnode over the same KV slice, so the
    cost is that of the sampled requests' own paths.  ``q`` holds the sampled requests only, in
    order; ``remap`` translates pool slots when ``k_pool`` / ``v_pool`` hold only the rows the
    sample needs.  Returns ``o [len(sample), Hq, D]`` in ``q.dtype``."""
    kv_entries, kv_offs, kv_lens, q_entries, q_offs, q_lens, req_entries, req_offs, req_lens = lists
    kv_entries = np.asarray(kv_entries).reshape(-1)
    vnode_by_row = np.empty(len(q_entries), dtype=np.int64)
    for v in range(len(q_offs)):
        vnode_by_row[q_offs[v]: q_offs[v] + q_lens[v]] = v
    new_entries, new_kv_offs, new_kv_lens, new_q = [], [], [], []
    r_entries, r_offs, r_lens = [], [], []
    for i, r in enumerate(sample):
        rows = req_entries[req_offs[r]: req_offs[r] + req_lens[r]]
        r_offs.append(len(new_q))
        r_lens.append(len(rows))
        for row in rows:
            assert q_entries[row] == r, "a request's list names a scratch row of another request"
            v = vnode_by_row[row]
            slots = kv_entries[kv_offs[v]: kv_offs[v] + kv_lens[v]]
            if remap is not None:
                slots = [remap[int(s)] for s in slots]
            new_kv_offs.append(len(new_entries))
            new_kv_lens.append(len(slots))
            new_entries.extend(int(s) for s in slots)
            r_entries.append(len(new_q))
            new_q.append(i)
    n = len(new_q)
    mid_o, mid_lse = stage1_arith(q, k_pool, v_pool, np.asarray(new_entries, dtype=np.int64), new_kv_offs,
                                  new_kv_lens, new_q, list(range(n)), [1] * n, kv_tile, sm_scale, n)
    return stage2_arith(r_entries, r_offs, r_lens, mid_o, mid_lse, q.dtype)


def gathered_attention_torch(q, k_pool, v_pool, path_tokens, sm_scale, requests=None):
    """The reference's no-sharing formulation on the CPU: per request, gather the path KV
    from the pool and attend with PyTorch fp32 ops.  ``requests`` limits the work to a
    sample (the bench's bounded CPU baseline)."""
    batch, hq, d = q.shape
    hkv = k_pool.shape[1]
    g = hq // hkv
    picks = range(batch) if requests is None else requests
    out = torch.zeros((batch, hq, d), dtype=torch.float32)
    for r in picks:
        idx = torch.as_tensor(np.asarray(path_tokens[r]), dtype=torch.long)
        k = k_pool[idx].to(torch.float32).permute(1, 0, 2)       # [Hkv, L, D]
        v = v_pool[idx].to(torch.float32).permute(1, 0, 2)
        qr = q[r].to(torch.float32).view(hkv, g, d)
        prob = torch.softmax(torch.bmm(qr, k.transpose(1, 2)) * sm_scale, dim=-1)
        out[r] = torch.bmm(prob, v).reshape(hq, d)
    return out


# ----------------------------------------------------------------------------------------
# planner restatement (integers and IEEE doubles only)
# ----------------------------------------------------------------------------------------

class PlanResult:
    pass


def _pad_q(ts, n):
    return ts - ((n - 1) % ts + 1)          # fasttree.py:30-31, Python floor modulo


def _mm(nq, nk, P):
    ph = 0 if nq > P["TSQs"][1] else 1      # fasttree.py:38-45, evaluated left to right
    return (P["alpha"] * _pad_q(P["TSQs"][ph], nq) * P["g"] * nk
            + P["beta"] * max(0, P["TSKs"][ph] - nk) * nq * P["g"])


def _split_decisions(parent, seqlen, nreq, P):
    """fasttree.py:64-96."""
    n = len(parent)
    kids = [[] for _ in range(n)]
    for i in range(1, n):
        kids[parent[i]].append(i)
    run = list(seqlen)
    take = [0] * n
    todo = deque([0])
    while todo:
        v = todo.popleft()
        here = nreq[v]
        for l in kids[v]:
            c_k = _mm(here, run[v], P) + _mm(nreq[l], run[l], P) + P["gamma"] * nreq[l]
            c_q = _mm(here - nreq[l], run[v], P) + _mm(nreq[l], run[l] + run[v], P)
            if c_k > c_q:
                take[l] = 1
                here -= nreq[l]
                run[l] = run[l] + run[v]
            todo.append(l)
    return take


def plan(parent: List[int], seqlen: List[int], nchild: List[int], requests: List[List[int]],
         kv_ptrs: List[int], batch: int, hkv: int, alpha, beta, gamma, TSQs, TSKs, g,
         kv_split_sizes, thr1, thr2) -> PlanResult:
    """fasttree.py:111-262 restated over plain lists.  ``TSQs``/``TSKs`` are not mutated;
    their final values are returned on the result."""
    n = len(parent)
    P = dict(alpha=alpha, beta=beta, gamma=gamma, TSQs=list(TSQs), TSKs=list(TSKs), g=g)
    nreq = [len(r) for r in requests]
    qt = list(TSQs)
    split = [kv_split_sizes[0], kv_split_sizes[0]]
    log = []

    def survey(take):
        served = [[] for _ in range(n)]
        fifo = deque(i for i in range(n) if nchild[i] == 0)
        for i in fifo:
            served[i] = list(requests[i])
        left = list(nchild)
        while fifo:
            i = fifo.popleft()
            if take[i] == 0 and i != 0:
                served[parent[i]].extend(requests[i])
            left[parent[i]] -= 1                      # parent[0] == -1 hits the last slot
            if left[parent[i]] == 0:
                fifo.append(parent[i])
        para = [0, 0]
        for i in range(n):
            if not served[i]:
                continue
            length, w = seqlen[i], i
            while take[w] == 1:
                w = parent[w]
                length += seqlen[w]
            ph = 0 if len(served[i]) > qt[1] else 1
            para[ph] += ((len(served[i]) - 1) // qt[ph] + 1) * ((length - 1) // split[ph] + 1)
        return served, [x * hkv for x in para]

    for attempt in range(3):
        take = _split_decisions(parent, seqlen, nreq, P)
        served, para = survey(take)
        log.append(f"parallelisms: {para}")
        if attempt == 0:
            low = [ph for ph in (0, 1) if 0 < para[ph] < thr1[ph]]
            for ph in low:
                split[ph] = kv_split_sizes[1]
            if not low:
                break
        elif attempt == 1:
            if 0 < para[0] < thr2[0]:
                qt = [qt[1], qt[1]]
                P["TSQs"], P["TSKs"] = qt, [P["TSKs"][1]] * 2
            elif 0 < para[1] < thr2[1]:
                qt = [qt[0], qt[0]]
                P["TSQs"], P["TSKs"] = qt, [P["TSKs"][0]] * 2
            else:
                break
    log += [str(qt), str(split)]

    kv_entries, kv_offs, kv_lens, q_entries, q_offs, q_lens = [], [], [], [], [], []
    for i in range(n):
        cnt = len(served[i])
        if cnt == 0:
            continue
        ks = split[0 if cnt > qt[1] else 1]
        chain, w = [i], i
        while take[w] == 1:
            w = parent[w]
            chain.insert(0, w)
        base = len(kv_entries)
        for node in chain:
            kv_entries.extend(range(kv_ptrs[node], kv_ptrs[node + 1]))
        length = len(kv_entries) - base
        for a in range((length - 1) // ks + 1):
            qbase = len(q_entries)
            q_entries.extend(served[i])
            for b in range((cnt - 1) // qt[0] + 1):
                kv_offs.append(base + a * ks)
                kv_lens.append(min((a + 1) * ks, length) - a * ks)
                q_offs.append(qbase + b * qt[0])
                q_lens.append(min((b + 1) * qt[0], cnt) - b * qt[0])

    per_req = [[] for _ in range(batch)]
    for row, r in enumerate(q_entries):
        per_req[r].append(row)
    req_offs = [0] * batch
    for r in range(1, batch):
        req_offs[r] = req_offs[r - 1] + len(per_req[r - 1])
    order = sorted(range(len(q_lens)), key=lambda v: q_lens[v] <= qt[1])   # stable: wide first
    wide = sum(1 for x in q_lens if x > qt[1])
    log += [f"Above threshold:  {wide}", f"Below threshold:  {len(q_lens) - wide}"]

    res = PlanResult()
    res.vnode_to_kv_entries = kv_entries + [-1] * 32
    res.vnode_to_kv_offs = [kv_offs[v] for v in order]
    res.vnode_to_kv_lens = [kv_lens[v] for v in order]
    res.vnode_to_q_entries = q_entries
    res.vnode_to_q_offs = [q_offs[v] for v in order]
    res.vnode_to_q_lens = [q_lens[v] for v in order]
    res.req_to_vnode_entries = [row for rows in per_req for row in rows] + [-1] * 32
    res.req_to_vnode_offs = req_offs
    res.req_to_vnode_lens = [len(rows) for rows in per_req]
    res.phase_node_nums = [wide, len(q_lens) - wide]
    res.phase_node_offsets = [0, wide]
    res.node_assignments = take
    res.final_TSQs, res.final_TSKs = list(P["TSQs"]), list(P["TSKs"])
    res.stdout = "\n".join(log) + "\n"
    return res


def plan_from_tree(tree_info, kv_ptrs, batch, case) -> PlanResult:
    """Convenience wrapper over node objects and a tests/golden case record."""
    return plan(
        [t.parent for t in tree_info], [t.seqlen for t in tree_info], [t.num_children for t in tree_info],
        [list(t.requests) for t in tree_info], list(kv_ptrs), batch, case["Hkv"],
        case["alpha"], case["beta"], case["gamma"], case["TSQs"], case["TSKs"], case["Hq"] // case["Hkv"],
        case["kv_split_sizes"], case["para_threshs1"], case["para_threshs2"])
