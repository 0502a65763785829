"""Host-side planner of FastTree decode attention: cost model, greedy tree splitter,
adaptive parallelism loop and the virtual-node ("vnode") metadata builder.

The planner decides, for every radix-tree node, whether its KV is attended together
with its parent's KV by the node's own requests only (``assignment 1``: the child
absorbs the ancestor KV, a "Q split") or whether the parent keeps one shared pass
for all of its requests and the child adds a separate partial (``assignment 0``: a
"K split" whose price is one more partial to merge).  It then cuts every resulting
(query set, KV run) pair into vnodes of at most ``Q_TILE`` queries and
``KV_SPLIT`` tokens and emits the index arrays the two device kernels walk.

Every list this module produces is element-for-element identical to what the
reference planner produces for the same arguments, including its mutation of the
``FastTreeParams`` object and the lines it prints.

Reference: kernel_bench/fasttree.py:7-27 (parameters), :30-61 (cost model),
:64-96 (greedy splitter), :99-296 (adaptive loop and metadata builder).
"""

from __future__ import annotations

import os
from collections import deque
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import _plan_lib

#: The reference prints its parallelism estimates, final tile/split sizes and the
#: per-phase vnode counts on every call.  Set to False to silence the planner.
VERBOSE = True

#: Which implementation ``fasttree_plan`` runs: "native" (libfasttree_plan.so, the C++ planner
#: behind include/fasttree_plan.h), "python" (this module), or "auto": native when the library is
#: built and the arguments fit its 32-bit interface.  Both produce identical plans.
BACKEND = os.environ.get("FASTTREE_PLANNER", "auto")

#: Number of -1 entries appended to the two entry arrays (kernel_bench/fasttree.py:261-262).
ENTRY_PADDING = 32


class FastTreeParams:
    """Mutable hyper-parameters of the cost model (kernel_bench/fasttree.py:7-27).

    ``fasttree_preparation`` may replace ``TSQs``/``TSKs`` through the setters while
    it adapts the tile sizes; callers that reuse one object across trees see that.
    """

    alpha = 0.66
    beta = 0.33
    gamma = 0.1
    TSQs = [64, 16]
    TSKs = [32, 128]
    kv_group_num = 1

    def set_values(self, alpha, beta, gamma):
        self.alpha, self.beta, self.gamma = alpha, beta, gamma

    def set_kv_group_num(self, kv_group_num):
        self.kv_group_num = kv_group_num

    def set_q_tile_sizes(self, TSQs):
        self.TSQs = TSQs

    def set_kv_tile_sizes(self, TSKs):
        self.TSKs = TSKs


# --------------------------------------------------------------------------------------
# Cost model.  All arithmetic is Python int / IEEE double evaluated left to right,
# exactly as in the reference, so that near-tie decisions come out the same.
# --------------------------------------------------------------------------------------

def _CpadQ(TS, N):
    """Query rows wasted when N queries are tiled by TS (kernel_bench/fasttree.py:30-31).
    Python's floor modulo makes N == 0 cost nothing: (-1) % TS == TS - 1."""
    return TS - ((N - 1) % TS + 1)


def _CpadK(TS, N):
    """KV columns wasted when fewer than one tile of keys exists (fasttree.py:34-35)."""
    return max(0, TS - N)


def _Cmm(nQ, nK, params: FastTreeParams):
    """Padding cost of one (nQ queries x nK keys) contraction (fasttree.py:38-45)."""
    phase = 0 if nQ > params.TSQs[1] else 1
    tsq, tsk = params.TSQs[phase], params.TSKs[phase]
    q_waste = params.alpha * _CpadQ(tsq, nQ) * params.kv_group_num * nK
    k_waste = params.beta * _CpadK(tsk, nK) * nQ * params.kv_group_num
    return q_waste + k_waste


def _Cred(nQl, params: FastTreeParams, lenl, lenv):
    """Cost of merging one more partial per query (fasttree.py:48-49)."""
    return params.gamma * nQl


def _SplitQCost(nQcurr, nQl, lenv, lenl, params: FastTreeParams):
    """Child l leaves with its queries and a private copy of the parent's run
    (fasttree.py:52-53)."""
    return _Cmm(nQcurr - nQl, lenv, params) + _Cmm(nQl, lenl + lenv, params)


def _SplitKCost(nQcurr, nQl, lenl, lenv, params: FastTreeParams):
    """Parent run stays shared; child l is a separate partial (fasttree.py:56-61)."""
    return _Cmm(nQcurr, lenv, params) + _Cmm(nQl, lenl, params) + _Cred(nQl, params, lenl, lenv)


def _tree_heuristic(tree_info, params: FastTreeParams) -> List[int]:
    """Greedy top-down split decision per node (kernel_bench/fasttree.py:64-96).

    Nodes are visited breadth first from node 0, children in ascending id.  While a
    node's children are scanned, the number of queries still attached to the node
    shrinks by every child that took the Q split, and a child that took it carries the
    accumulated run length down to its own children.
    """
    count = len(tree_info)
    children: List[List[int]] = [[] for _ in range(count)]
    for nid in range(1, count):
        children[tree_info[nid].parent].append(nid)
    run_len = [tree_info[nid].seqlen for nid in range(count)]

    assignment = [0] * count
    pending = deque([0])
    while pending:
        v = pending.popleft()
        attached = len(tree_info[v].requests)
        lenv = run_len[v]
        for l in children[v]:
            nQl = len(tree_info[l].requests)
            lenl = run_len[l]
            keep_shared = _SplitKCost(attached, nQl, lenl, lenv, params)
            go_private = _SplitQCost(attached, nQl, lenv, lenl, params)
            if keep_shared > go_private:
                assignment[l] = 1
                attached -= nQl
                run_len[l] = lenl + lenv
            pending.append(l)
    return assignment


# --------------------------------------------------------------------------------------
# Plan: the pure-host result of the planner (python lists / numpy arrays only).
# --------------------------------------------------------------------------------------

@dataclass
class FastTreePlan:
    """Everything ``fasttree_preparation`` computes before it touches a device."""

    vnode_to_kv_entries: np.ndarray          # int32, padded with ENTRY_PADDING x -1
    vnode_to_kv_offs: List[int]
    vnode_to_kv_lens: List[int]
    vnode_to_q_entries: List[int]
    vnode_to_q_offs: List[int]
    vnode_to_q_lens: List[int]
    req_to_vnode_entries: List[int]          # padded with ENTRY_PADDING x -1
    req_to_vnode_offs: List[int]
    req_to_vnode_lens: List[int]
    phase_node_nums: List[int]
    phase_node_offsets: List[int]
    node_assignments: List[int]
    q_tile_sizes: List[int]                  # final Q_TILE_SIZE_PER_PHASE
    kv_split_sizes: List[int]                # final KV_SPLIT_SIZE_PER_PHASE
    parallelisms: List[List[int]] = field(default_factory=list)  # one entry per loop pass

    @property
    def num_rows(self) -> int:
        """Rows of the partial-result scratch (``mid_o.shape[0]``)."""
        return len(self.vnode_to_q_entries)

    @property
    def num_vnodes(self) -> int:
        return len(self.vnode_to_q_lens)


def _say(*args):
    if VERBOSE:
        print(*args)


def _requests_per_node(tree_info, assignment) -> List[List[int]]:
    """Which requests each node's own vnodes serve (fasttree.py:126-141).

    Leaves start with their own request list.  Nodes are then retired in a FIFO order
    (all leaves in ascending id first, a parent as soon as its last child retires); a
    retiring node that did not take the Q split hands *all* requests below it to its
    parent, in retirement order.  The root's parent is -1, which Python resolves to
    the last list element; the reference does the same and nothing depends on it.
    """
    count = len(tree_info)
    served: List[List[int]] = [[] for _ in range(count)]
    fifo = deque()
    for nid in range(count):
        if tree_info[nid].num_children == 0:
            fifo.append(nid)
            served[nid] = list(tree_info[nid].requests)
    waiting = [tree_info[nid].num_children for nid in range(count)]
    while fifo:
        nid = fifo.popleft()
        up = tree_info[nid].parent
        if assignment[nid] == 0 and nid != 0:
            served[up] += tree_info[nid].requests
        waiting[up] -= 1
        if waiting[up] == 0:
            fifo.append(up)
    return served


def _run_chain(tree_info, assignment, nid) -> Tuple[List[int], int]:
    """Nodes whose KV the vnodes of ``nid`` attend, ancestors first, and the run length
    (fasttree.py:149-153, :202-210)."""
    chain = [nid]
    total = tree_info[nid].seqlen
    walk = nid
    while assignment[walk] == 1:
        walk = tree_info[walk].parent
        chain.append(walk)
        total += tree_info[walk].seqlen
    chain.reverse()
    return chain, total


def _estimate_parallelism(tree_info, assignment, served, q_tiles, kv_splits, num_kv_heads):
    """Thread-block count per phase the current plan would launch (fasttree.py:143-159)."""
    blocks = [0, 0]
    for nid, reqs in enumerate(served):
        n = len(reqs)
        if n == 0:
            continue
        _, kv_len = _run_chain(tree_info, assignment, nid)
        phase = 0 if n > q_tiles[1] else 1
        blocks[phase] += ((kv_len - 1) // kv_splits[phase] + 1) * ((n - 1) // q_tiles[phase] + 1)
    return [b * num_kv_heads for b in blocks]


def _fits_native(KV_ptrs, KV_SPLIT_SIZES, para_threshs1, para_threshs2, params) -> bool:
    """The native planner takes tile sizes, split sizes, thresholds and token positions as int32."""
    limit = 2 ** 31 - 1 - ENTRY_PADDING
    small = [*KV_SPLIT_SIZES[:2], *para_threshs1[:2], *para_threshs2[:2], *params.TSQs[:2], *params.TSKs[:2],
             params.kv_group_num]
    return (all(isinstance(x, (int, np.integer)) and 1 <= x <= limit for x in small[:2] + small[6:])
            and all(isinstance(x, (int, np.integer)) and -limit <= x <= limit for x in small[2:6])
            and len(KV_ptrs) > 0 and int(KV_ptrs[-1]) <= limit)


def _plan_native(tree_info, KV_ptrs, batch_size, num_kv_heads, KV_SPLIT_SIZES, para_threshs1, para_threshs2,
                 params: FastTreeParams, kv_slot_map) -> FastTreePlan:
    """``fasttree_plan`` through libfasttree_plan.so: same result, same printed lines, same
    replacement of ``params.TSQs`` / ``params.TSKs`` when the second adaptation pass fires."""
    L = _plan_lib
    r = L.plan(tree_info, KV_ptrs, batch_size, num_kv_heads, KV_SPLIT_SIZES, para_threshs1, para_threshs2,
               params.alpha, params.beta, params.gamma, params.TSQs, params.TSKs, params.kv_group_num,
               kv_slot_map=kv_slot_map)
    history = r[L.PARALLELISMS].reshape(-1, 2).tolist()
    for para in history:
        _say("parallelisms:", para)
    q_tiles = r[L.Q_TILE_SIZES].tolist()
    if int(r[L.TILES_REPLACED][0]):
        params.set_q_tile_sizes(q_tiles)
        params.set_kv_tile_sizes(r[L.KV_TILE_SIZES].tolist())
    kv_splits = r[L.KV_SPLIT_SIZES].tolist()
    _say(q_tiles)
    _say(kv_splits)
    nums = r[L.PHASE_NODE_NUMS].tolist()
    _say("Above threshold: ", nums[0])
    _say("Below threshold: ", nums[1])
    return FastTreePlan(
        vnode_to_kv_entries=r[L.KV_ENTRIES],
        vnode_to_kv_offs=r[L.KV_OFFS].tolist(),
        vnode_to_kv_lens=r[L.KV_LENS].tolist(),
        vnode_to_q_entries=r[L.Q_ENTRIES].tolist(),
        vnode_to_q_offs=r[L.Q_OFFS].tolist(),
        vnode_to_q_lens=r[L.Q_LENS].tolist(),
        req_to_vnode_entries=r[L.REQ_ENTRIES].tolist(),
        req_to_vnode_offs=r[L.REQ_OFFS].tolist(),
        req_to_vnode_lens=r[L.REQ_LENS].tolist(),
        phase_node_nums=nums,
        phase_node_offsets=r[L.PHASE_NODE_OFFSETS].tolist(),
        node_assignments=r[L.NODE_ASSIGNMENTS].tolist(),
        q_tile_sizes=list(q_tiles),
        kv_split_sizes=kv_splits,
        parallelisms=history,
    )


def fasttree_plan(
    tree_info,
    KV_ptrs: Sequence[int],
    batch_size: int,
    num_kv_heads: int,
    KV_SPLIT_SIZES: Sequence[int],
    para_threshs1: Sequence[int],
    para_threshs2: Sequence[int],
    params: FastTreeParams,
    kv_slot_map: Optional[np.ndarray] = None,
    backend: Optional[str] = None,
) -> FastTreePlan:
    """Run the planner and return host-side lists (kernel_bench/fasttree.py:111-262).

    ``backend`` overrides the module's ``BACKEND`` for this call.

    ``kv_slot_map`` (optional, length ``KV_ptrs[-1]``) maps the logical token position
    ``KV_ptrs[node] + t`` to the slot of the KV pool that holds it; without it the pool
    is node-major and the entries are the logical positions themselves, as in the
    reference's bench.
    """
    choice = backend or BACKEND
    if choice == "native" or (choice == "auto" and _plan_lib.available() and _fits_native(
            KV_ptrs, KV_SPLIT_SIZES, para_threshs1, para_threshs2, params)):
        return _plan_native(tree_info, KV_ptrs, batch_size, num_kv_heads, KV_SPLIT_SIZES, para_threshs1,
                            para_threshs2, params, kv_slot_map)

    count = len(tree_info)
    q_tiles = params.TSQs                       # alias on purpose, as in the reference
    kv_splits = [KV_SPLIT_SIZES[0], KV_SPLIT_SIZES[0]]
    history: List[List[int]] = []

    # Up to three passes: (0) shrink KV splits of under-parallel phases, (1) collapse
    # both phases onto one tile shape if still under-parallel, (2) re-plan with those.
    for attempt in range(3):
        assignment = _tree_heuristic(tree_info, params)
        served = _requests_per_node(tree_info, assignment)
        para = _estimate_parallelism(tree_info, assignment, served, q_tiles, kv_splits, num_kv_heads)
        history.append(para)
        _say("parallelisms:", para)
        if attempt == 0:
            starved = [ph for ph in range(2) if 0 < para[ph] < para_threshs1[ph]]
            for ph in starved:
                kv_splits[ph] = KV_SPLIT_SIZES[1]
            if not starved:
                break
        elif attempt == 1:
            if 0 < para[0] < para_threshs2[0]:
                keep = 1
            elif 0 < para[1] < para_threshs2[1]:
                keep = 0
            else:
                break
            q_tiles = [q_tiles[keep], q_tiles[keep]]
            params.set_q_tile_sizes(q_tiles)
            params.set_kv_tile_sizes([params.TSKs[keep], params.TSKs[keep]])

    _say(q_tiles)
    _say(kv_splits)

    ptrs = np.asarray(KV_ptrs, dtype=np.int64)
    kv_runs: List[np.ndarray] = []
    kv_total = 0
    kv_offs: List[int] = []
    kv_lens: List[int] = []
    q_entries: List[int] = []
    q_offs: List[int] = []
    q_lens: List[int] = []

    q_tile = q_tiles[0]                         # phase-0 tile for every node (fasttree.py:194)
    for nid in range(count):
        reqs = served[nid]
        n = len(reqs)
        if n == 0:
            continue
        kv_split = kv_splits[0 if n > q_tiles[1] else 1]
        chain, kv_len = _run_chain(tree_info, assignment, nid)
        run_base = kv_total
        for member in chain:
            kv_runs.append(np.arange(ptrs[member], ptrs[member + 1], dtype=np.int64))
        kv_total += kv_len

        for kv_lo in range(0, kv_len, kv_split):
            row_base = len(q_entries)
            q_entries.extend(reqs)              # one scratch row per (request, kv split)
            span = min(kv_lo + kv_split, kv_len) - kv_lo
            for q_lo in range(0, n, q_tile):
                kv_offs.append(run_base + kv_lo)
                kv_lens.append(span)
                q_offs.append(row_base + q_lo)
                q_lens.append(min(q_lo + q_tile, n) - q_lo)

    rows_of_req: List[List[int]] = [[] for _ in range(batch_size)]
    for row, req in enumerate(q_entries):
        rows_of_req[req].append(row)
    req_offs: List[int] = []
    req_lens: List[int] = []
    req_entries: List[int] = []
    for rows in rows_of_req:
        req_offs.append(len(req_entries))
        req_lens.append(len(rows))
        req_entries.extend(rows)

    # Stable partition: vnodes wider than the small tile run first (phase 0).
    small = q_tiles[1]
    wide = [v for v, n in enumerate(q_lens) if n > small]
    narrow = [v for v, n in enumerate(q_lens) if n <= small]
    _say("Above threshold: ", len(wide))
    _say("Below threshold: ", len(narrow))
    order = wide + narrow

    logical = np.concatenate(kv_runs) if kv_runs else np.zeros(0, dtype=np.int64)
    if kv_slot_map is not None:
        logical = np.asarray(kv_slot_map)[logical]
    padded = np.concatenate([logical, np.full(ENTRY_PADDING, -1, dtype=np.int64)]).astype(np.int32)

    return FastTreePlan(
        vnode_to_kv_entries=padded,
        vnode_to_kv_offs=[kv_offs[v] for v in order],
        vnode_to_kv_lens=[kv_lens[v] for v in order],
        vnode_to_q_entries=q_entries,
        vnode_to_q_offs=[q_offs[v] for v in order],
        vnode_to_q_lens=[q_lens[v] for v in order],
        req_to_vnode_entries=req_entries + [-1] * ENTRY_PADDING,
        req_to_vnode_offs=req_offs,
        req_to_vnode_lens=req_lens,
        phase_node_nums=[len(wide), len(narrow)],
        phase_node_offsets=[0, len(wide)],
        node_assignments=assignment,
        q_tile_sizes=list(q_tiles),
        kv_split_sizes=kv_splits,
        parallelisms=history,
    )


class PlanBuffers:
    """Device buffers for :func:`fasttree_preparation`, allocated once at stated maxima and
    filled in place by every call that is given them: a serving loop re-plans whenever its batch
    changes, and neither the nine index arrays nor the fp32 scratch should be allocated anew each
    time (the reference says so of its own bench code, kernel_bench/fasttree.py:264, and
    pre-allocates in its plugin, metadata.py:40-58).

    ``max_kv_entries`` bounds the flat KV index list (unique tokens plus what merged chains
    replicate, plus the 32 padding entries), ``max_rows`` the scratch rows (one per request and
    KV split), ``max_vnodes`` the vnodes, ``max_batch_size`` the requests.
    """

    def __init__(self, num_qo_heads, head_dim, max_kv_entries, max_rows, max_vnodes, max_batch_size, device="cuda"):
        import torch

        def ints(n):
            return torch.empty(int(n), dtype=torch.int32, device=device)

        self.device = device
        self.vnode_to_kv_entries = ints(max_kv_entries)
        self.vnode_to_kv_offs, self.vnode_to_kv_lens = ints(max_vnodes), ints(max_vnodes)
        self.vnode_to_q_entries = ints(max_rows)
        self.vnode_to_q_offs, self.vnode_to_q_lens = ints(max_vnodes), ints(max_vnodes)
        self.req_to_vnode_entries = ints(max_rows + 32)
        self.req_to_vnode_offs, self.req_to_vnode_lens = ints(max_batch_size), ints(max_batch_size)
        self.prog_table = ints(4 * max_vnodes)
        self.narrow_table = ints(64 * max_vnodes)     # (launch_schedule.NARROW_RECORD entries per narrow vnode)
        self.req_table = ints(16 * max_batch_size)    # (launch_schedule.REQUEST_RECORD entries per request)
        self.prog_records = ints(256 * max_vnodes)    # (launch_schedule.PROGRAM_RECORD entries per program)
        self.mid_o = torch.empty((int(max_rows), num_qo_heads, head_dim), dtype=torch.float32, device=device)
        self.mid_lse = torch.empty((int(max_rows), num_qo_heads), dtype=torch.float32, device=device)

    def fill(self, name, values):
        """Copies ``values`` into the front of buffer ``name`` and returns that part of it."""
        import torch

        host = torch.from_numpy(np.ascontiguousarray(np.asarray(values, dtype=np.int32)))
        dst = getattr(self, name)
        if host.numel() > dst.numel():
            raise ValueError(f"{name}: {host.numel()} entries do not fit the {dst.numel()} that were allocated")
        part = dst[: host.numel()]
        part.copy_(host)
        return part


def place_plan(kv_entries, vnodes, q_entries, per_request, phase_nums, phase_offs,
               batch_size, num_qo_heads, num_kv_heads, head_dim, *,
               device="cuda", launch_order=False, buffers=None, num_cus=None):
    """The 13 arguments ``fasttree_decode`` takes after the output tensor, from vnode lists on the
    host: ``kv_entries`` (flat pool slots), ``vnodes = (kv_offs, kv_lens, q_offs, q_lens)``,
    ``q_entries`` (request of every scratch row), ``per_request = (entries, offs, lens)`` (scratch
    rows of every request; ignored with ``launch_order``, which derives its own), the two phase
    lists.  Places the nine int32 arrays and the two fp32 partial-result buffers on ``device`` (into
    ``buffers`` if given).  With ``launch_order`` the lists are first arranged as block programs
    (:func:`launch_schedule.block_programs`) for ``num_cus`` compute units, and ``phase_node_nums``
    comes back as a list that also carries the program table and the host-written records."""
    import torch

    from .launch_schedule import LaunchPhases, block_programs

    names = iter(("vnode_to_kv_entries", "vnode_to_kv_offs", "vnode_to_kv_lens", "vnode_to_q_entries", "vnode_to_q_offs",
                  "vnode_to_q_lens", "req_to_vnode_entries", "req_to_vnode_offs", "req_to_vnode_lens"))

    def place(name, values):
        if buffers is not None:
            return buffers.fill(name, values)
        host = torch.from_numpy(np.ascontiguousarray(np.asarray(values, dtype=np.int32)))
        return host.to(device)

    def put(values):
        return place(next(names), values)  # (the nine arrays are placed in this order below)

    rows = int(len(np.asarray(q_entries).reshape(-1)))
    if launch_order:
        group = max(1, num_qo_heads // num_kv_heads)
        if num_cus is None:
            from .launch_schedule import compute_units
            num_cus = compute_units(device)
        sched = block_programs(*vnodes, q_entries, batch_size, group, num_kv_heads, head_dim=head_dim, num_cus=num_cus)
        vnodes = (sched.kv_offs, sched.kv_lens, sched.q_offs, sched.q_lens)
        q_entries = sched.q_entries
        per_request = (sched.req_entries, sched.req_offs, sched.req_lens)
        rows = sched.num_rows
        phase_nums, phase_offs = LaunchPhases(sched.phase_node_nums), list(sched.phase_node_offsets)
        phase_nums.modelled_us, phase_nums.num_cus, phase_nums.block_slots = sched.modelled_us, sched.num_cus, sched.block_slots
        if sched.num_programs > 0:
            phase_nums.prog_table = place("prog_table", sched.prog_table.reshape(-1))
            phase_nums.num_programs = sched.num_programs
            phase_nums.narrow_in_programs = sched.narrow_in_programs
        from . import launch_schedule
        if sched.num_programs > 0 and head_dim >= 32 and launch_schedule.USE_PROGRAM_RECORDS:
            records = launch_schedule.program_records(kv_entries, *vnodes, q_entries, sched.prog_table,
                                                      phase_offs[0], group)
            phase_nums.prog_records = place("prog_records", records.reshape(-1))
        if phase_nums[1] > 0 and head_dim >= 32 and launch_schedule.USE_NARROW_RECORDS:
            from .launch_schedule import narrow_records
            records = narrow_records(kv_entries, *vnodes, q_entries, phase_offs[1], phase_nums[1])
            phase_nums.narrow_table = place("narrow_table", records.reshape(-1))
        if head_dim >= 32 and launch_schedule.USE_REQUEST_RECORDS:
            from .launch_schedule import request_records
            phase_nums.req_table = place("req_table", request_records(*per_request).reshape(-1))
    if buffers is not None:
        if rows > buffers.mid_o.shape[0] or buffers.mid_o.shape[1:] != (num_qo_heads, head_dim):
            raise ValueError(f"the scratch of the buffers ({tuple(buffers.mid_o.shape)}) does not hold "
                             f"{rows} rows of {num_qo_heads} x {head_dim}")
        mid_o, mid_lse = buffers.mid_o[:rows], buffers.mid_lse[:rows]
    else:
        mid_o = torch.empty((rows, num_qo_heads, head_dim), dtype=torch.float32, device=device)
        mid_lse = torch.empty((rows, num_qo_heads), dtype=torch.float32, device=device)
    return (
        put(kv_entries),
        put(vnodes[0]),
        put(vnodes[1]),
        put(q_entries),
        put(vnodes[2]),
        put(vnodes[3]),
        put(per_request[0]),
        put(per_request[1]),
        put(per_request[2]),
        mid_o,
        mid_lse,
        phase_nums,
        phase_offs,
    )


def fasttree_preparation(
    tree_info,
    KV_ptrs,
    batch_size,
    num_qo_heads,
    num_kv_heads,
    head_dim,
    KV_SPLIT_SIZES,
    para_threshs1,
    para_threshs2,
    params: FastTreeParams,
    *,
    device="cuda",
    kv_slot_map=None,
    launch_order=False,
    buffers=None,
    num_cus=None,
):
    """Drop-in for kernel_bench/fasttree.py:99-296: plan on the host, then place the nine
    int32 index arrays and the two fp32 partial-result buffers on ``device``.

    Returns ``((vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens,
    vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, req_to_vnode_entries,
    req_to_vnode_offs, req_to_vnode_lens, mid_o, mid_lse, phase_node_nums,
    phase_node_offsets), node_assignments)``: element for element the reference's lists.

    The keyword-only arguments do not exist in the reference: ``device`` defaults to the
    reference's hard-wired "cuda"; ``kv_slot_map`` is described in :func:`fasttree_plan`; with
    ``buffers`` (a :class:`PlanBuffers`) nothing is allocated on the device: the arrays are
    written into its buffers and the returned tensors are their leading parts.  With
    ``launch_order=True`` the lists come back arranged for an MI355X instead
    (:func:`launch_schedule.block_programs`: the same computation as block programs,
    with scratch rows and per-request lists of its own); ``phase_node_nums`` is then a list that
    also carries the program table, which ``fasttree_decode`` picks up; the programs are laid out
    for ``num_cus`` compute units (None: those ``device`` reports, 256 where it is not a GPU).
    """
    plan = fasttree_plan(
        tree_info, KV_ptrs, batch_size, num_kv_heads,
        KV_SPLIT_SIZES, para_threshs1, para_threshs2, params, kv_slot_map=kv_slot_map,
    )

    aux = place_plan(
        plan.vnode_to_kv_entries,
        (plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens),
        plan.vnode_to_q_entries,
        (plan.req_to_vnode_entries, plan.req_to_vnode_offs, plan.req_to_vnode_lens),
        list(plan.phase_node_nums), list(plan.phase_node_offsets),
        batch_size, num_qo_heads, num_kv_heads, head_dim,
        device=device, launch_order=launch_order, buffers=buffers, num_cus=num_cus,
    )
    return aux, plan.node_assignments
