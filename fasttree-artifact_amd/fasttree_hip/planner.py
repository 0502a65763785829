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


#: A first-phase vnode of at most LIGHT_VNODE_ROWS query rows and LIGHT_VNODE_WORK query rows x
#: KV tokens is launched with the second phase when the first phase alone has more blocks than
#: WIDE_BLOCK_SLOTS, the number an MI355X runs at a time (256 compute units x 2); see
#: :func:`vnodes_in_launch_order`.
LIGHT_VNODE_WORK = 4096
LIGHT_VNODE_ROWS = 64
WIDE_BLOCK_SLOTS = 512


#: Query rows one block of the first-phase kernel serves per pass.
WIDE_BLOCK_ROWS = 128


def vnodes_in_launch_order(kv_offs, kv_lens, q_offs, q_lens, phase_node_nums, phase_node_offsets, group,
                           num_kv_heads=None, light_work=None, q_tile=None, return_order=False):
    """The four per-vnode lists and the two phase lists, rearranged for the decode kernels.

    A vnode is the tuple (kv_offs[v], kv_lens[v], q_offs[v], q_lens[v]); nothing else refers to
    a vnode by its position (the per-request lists of kernel_bench/fasttree.py:233-244 name
    scratch rows, not vnodes), and the kernels compute a vnode of any number of query rows in
    either phase, so the order within a phase and the phase a vnode is launched with change the
    schedule, not the result.  Three changes against the reference's order (fasttree.py:246-259):

    * light first-phase vnodes -- at most :data:`LIGHT_VNODE_ROWS` query rows and query rows x
      KV tokens at most ``light_work`` (default :data:`LIGHT_VNODE_WORK`) -- move to the second
      phase, provided the first phase has more blocks (vnodes x ``num_kv_heads``) than the
      machine runs at a time (:data:`WIDE_BLOCK_SLOTS`; always, when ``num_kv_heads`` is None).
      A first-phase vnode gets a block of four waves with a staging ring for long runs, two
      blocks per compute unit; a second-phase vnode gets one wave that serves 16 rows per
      pass, eight or more per compute unit.  Short runs under a few dozen rows are bound by
      memory latency, not by arithmetic: when there are more of them than block slots, they
      finish sooner with more of them in flight; when there are fewer, a block's four waves
      finish one sooner than a single wave's passes do.
    * the second phase is listed in order of decreasing work (KV tokens x passes of 16 rows;
      equal work keeps the order).  The kernel hands these vnodes to the machine in list order,
      each to one wave that walks its run tile by tile: a long run that starts last is what the
      launch then waits for.
    * with ``q_tile`` (the first phase's query tile, in requests) given: neighbours in the
      first phase that attend the same KV run with adjoining scratch rows -- the query tiles one
      node was cut into (fasttree.py:212-231) -- are joined into one vnode of at most
      ``WIDE_BLOCK_ROWS x ceil(q_tile x group / WIDE_BLOCK_ROWS)`` query rows, what the blocks of
      one vnode serve in a single pass: a tile of 16 requests x 4 heads fills half of a block's
      rows, and two such tiles would stage the same run twice.  Not done while the first phase
      has no more blocks than the machine has compute units (two half-filled blocks side by
      side finish sooner than one full block).  The kernel joins such neighbours itself when
      it is handed the reference's lists; joined here, no block is launched for the tiles
      that were absorbed.

    The order within the first phase is otherwise left alone (the kernel ranks those vnodes
    itself).  Returns ``(kv_offs, kv_lens, q_offs, q_lens, phase_node_nums, phase_node_offsets)``;
    with ``return_order`` a seventh element: for every vnode of the input its position in the
    output, or -1 for a query tile that was absorbed into its neighbour.
    """
    light_work = LIGHT_VNODE_WORK if light_work is None else light_work
    lists = [np.array(x, dtype=np.int32, copy=True) for x in (kv_offs, kv_lens, q_offs, q_lens)]
    first, count0, count1 = int(phase_node_offsets[0]), int(phase_node_nums[0]), int(phase_node_nums[1])
    if first != 0 or int(phase_node_offsets[1]) != count0:
        raise ValueError("the phases must be adjoining ranges starting at vnode 0")
    rows = lists[3].astype(np.int64) * int(group)
    tokens = lists[1].astype(np.int64)
    index = np.arange(count0 + count1)
    light = (index < count0) & (rows * tokens <= light_work) & (rows <= LIGHT_VNODE_ROWS)
    if num_kv_heads is not None and count0 * int(num_kv_heads) <= WIDE_BLOCK_SLOTS:
        light[:] = False
    wide = index[(index < count0) & ~light]
    narrow = np.concatenate([index[light], index[count0:]])
    work = tokens[narrow] * ((rows[narrow] + 15) // 16)
    narrow = narrow[np.argsort(-work, kind="stable")]
    order = np.concatenate([wide, narrow])
    lists = [x[order] for x in lists]
    n_wide = len(wide)
    kept_all = np.arange(len(order))
    if q_tile is not None and n_wide > 1:
        chunks = max(1, min(8, (int(q_tile) * int(group) + WIDE_BLOCK_ROWS - 1) // WIDE_BLOCK_ROWS))
        heads = 1 if num_kv_heads is None else int(num_kv_heads)
        if num_kv_heads is None or 2 * n_wide * heads * chunks > WIDE_BLOCK_SLOTS:
            cap = WIDE_BLOCK_ROWS * chunks // int(group)  # requests
            kept = [0]
            kv_o, kv_l, q_o, q_l = (x[:n_wide].astype(np.int64) for x in lists)
            q_l = q_l.copy()
            for v in range(1, n_wide):
                h = kept[-1]
                if (kv_o[v] == kv_o[h] and kv_l[v] == kv_l[h] and q_o[h] + q_l[h] == q_o[v]
                        and q_l[h] + q_l[v] <= cap):
                    q_l[h] += q_l[v]
                else:
                    kept.append(v)
            lists[3][:n_wide] = q_l.astype(np.int32)
            keep = np.concatenate([np.array(kept, dtype=np.int64), np.arange(n_wide, len(order))])
            lists = [x[keep] for x in lists]
            n_wide = len(kept)
            kept_all = keep
    result = (*lists, [n_wide, len(narrow)], [0, n_wide])
    if return_order:
        where = np.full(len(order), -1, dtype=np.int64)
        where[order[kept_all]] = np.arange(len(kept_all))
        result = (*result, where)
    return result


#: Blocks (128-row blocks x kv heads) the vnodes of one KV run must make for the run's KV split to
#: be undone: one per compute unit of an MI355X; see :func:`join_kv_chunks`.
FULL_MACHINE_BLOCKS = 256

#: First-phase blocks a launch may have for all of them to be resident at once with a few block
#: slots to spare (of :data:`WIDE_BLOCK_SLOTS`); see :func:`join_kv_chunks`.
RESIDENT_WIDE_BLOCKS = 472


def join_kv_chunks(kv_offs, kv_lens, q_offs, q_lens, q_entries, req_entries, req_offs, req_lens,
                   phase_node_nums, phase_node_offsets, group, num_kv_heads, min_blocks=None, resident_blocks=None,
                   return_order=False):
    """Cuts long KV runs into fewer chunks than the planner did where the chunks buy nothing.

    The planner cuts every run into chunks of the phase's KV split size whatever the number of
    requests under it (kernel_bench/fasttree.py:199-231): chunk s of a node is served by its own
    vnodes over its own copy of the node's scratch rows, and the second stage merges the copies
    per request.  The split buys parallelism, and each chunk costs a partial row per request and
    head to write, read and merge.  Two cases where fewer chunks are better:

    * a run attended by so many query rows that the 128-row blocks x kv heads of ONE chunk
      already number ``min_blocks`` (default :data:`FULL_MACHINE_BLOCKS`) has its parallelism
      without the split: it becomes one chunk;
    * a launch whose first phase has a few more blocks than the machine holds at once
      (``resident_blocks``, default :data:`RESIDENT_WIDE_BLOCKS`) runs its last blocks behind the
      others and keeps the second phase's short vnodes waiting for a block slot; when longer
      chunks bring the first phase under that number, the chunked runs are cut at the shortest
      common chunk length that does (C3: three chunks of its 4000-token root instead of four,
      472 blocks instead of 576).  Only runs whose blocks still number nine tenths of
      ``min_blocks`` afterwards are cut anew: a few long blocks on an otherwise idle machine
      would cost more.

    Where a vnode's KV slice ends the next chunk's begins (the flat KV index list holds a node's
    tokens back to back); vnodes over that next slice that serve the same requests in the same
    tiles are the next chunk.  A chain of S chunks that is to have S' < S is cut anew into S'
    equal slices (multiples of 64 tokens) served by the vnodes of its first S' chunks; the vnodes
    of the others are dropped together with their scratch rows, which leave the per-request
    lists (the rows stay allocated and unused).

    Takes the lists in the planner's order (first phase, then second) and returns
    ``(kv_offs, kv_lens, q_offs, q_lens, req_entries, req_offs, req_lens, phase_node_nums,
    phase_node_offsets)`` with ``req_entries`` padded by 32 x -1 as the planner's
    (fasttree.py:261-262); the inputs are not modified.  With ``return_order`` a tenth
    element: for every vnode of the input its position in the output, or -1 if it was dropped.
    """
    min_blocks = FULL_MACHINE_BLOCKS if min_blocks is None else int(min_blocks)
    resident = RESIDENT_WIDE_BLOCKS if resident_blocks is None else int(resident_blocks)
    kv_o, kv_l, q_o, q_l = (np.array(x, dtype=np.int64, copy=True) for x in (kv_offs, kv_lens, q_offs, q_lens))
    heads = max(1, int(num_kv_heads))
    count0 = int(phase_node_nums[0])
    n = len(kv_o)

    def unchanged():
        out = (kv_o.astype(np.int32), kv_l.astype(np.int32), q_o.astype(np.int32), q_l.astype(np.int32),
               np.asarray(req_entries, dtype=np.int32), np.asarray(req_offs, dtype=np.int32),
               np.asarray(req_lens, dtype=np.int32), list(phase_node_nums), list(phase_node_offsets))
        return (*out, np.arange(n, dtype=np.int64)) if return_order else out

    if n == 0:
        return unchanged()
    # blocks per run (the vnodes over one KV slice): requests summed over its vnodes
    _, first_of, run_of = np.unique((kv_o << 32) | kv_l, return_index=True, return_inverse=True)
    run_rows = np.bincount(run_of, weights=q_l).astype(np.int64) * int(group)
    run_blocks = -(-run_rows // WIDE_BLOCK_ROWS) * heads
    wide_total = int(run_blocks[first_of < count0].sum())  # (a run's vnodes share a phase but for a narrow last tile)
    full = run_blocks >= min_blocks
    if not full.any() and wide_total <= resident:
        return unchanged()
    # candidates: runs that another run follows or that follow another run
    run_start, run_end = kv_o[first_of], kv_o[first_of] + kv_l[first_of]
    chained = np.isin(run_end, run_start) | np.isin(run_start, run_end)
    if not chained.any():
        return unchanged()
    q_ent = np.asarray(q_entries, dtype=np.int64)
    runs = {}
    for v in np.nonzero(chained[run_of])[0].tolist():
        runs.setdefault((int(kv_o[v]), int(kv_l[v])), []).append(v)
    starts = {}
    for key in runs:
        starts.setdefault(key[0], []).append(key)
    chains, taken = [], set()
    for key in sorted(runs):
        if key in taken:
            continue
        chain, tiles, end = [key], runs[key], key[0] + key[1]
        while True:
            follower = None
            for cand in starts.get(end, ()):
                other = runs[cand]
                if cand in taken or cand == key or len(other) != len(tiles):
                    continue
                if all(q_l[a] == q_l[b] and (a < count0) == (b < count0)
                       and np.array_equal(q_ent[q_o[a]: q_o[a] + q_l[a]], q_ent[q_o[b]: q_o[b] + q_l[b]])
                       for a, b in zip(tiles, other)):
                    follower = cand
                    break
            if follower is None:
                break
            taken.add(follower)
            chain.append(follower)
            end = follower[0] + follower[1]
        if len(chain) > 1:
            rows = int(q_l[tiles].sum()) * int(group)
            chains.append((-(-rows // WIDE_BLOCK_ROWS) * heads, chain))
    # how many chunks each chain keeps
    plan = []
    for per, chain in chains:
        if per >= min_blocks:
            plan.append((per, chain, 1))
            if runs[chain[0]][0] < count0:
                wide_total -= per * (len(chain) - 1)
    if wide_total > resident:
        # One chunk length for all: the shortest for which the phase fits, every run that is cut
        # anew still covering the machine by itself (its blocks number nine tenths of min_blocks
        # or more; runs that cannot are left as they are -- a few long blocks on an otherwise
        # idle machine would be what the launch waits for).
        covering = max(1, 9 * min_blocks // 10)
        rest = []
        for per, chain in chains:
            fewest = -(-covering // per)
            if per < min_blocks and runs[chain[0]][0] < count0 and fewest < len(chain):
                rest.append((per, chain, sum(key[1] for key in chain), fewest))
        fixed = wide_total - sum(per * len(chain) for per, chain, _, _ in rest)

        def chunks_at(length):
            return [min(len(chain), max(fewest, -(-tokens // length))) for _, chain, tokens, fewest in rest]

        lengths = sorted({-(-tokens // k) for _, chain, tokens, fewest in rest for k in range(fewest, len(chain) + 1)})
        for length in lengths:
            keeps = chunks_at(length)
            if fixed + sum(per * keep for (per, _, _, _), keep in zip(rest, keeps)) <= resident:
                plan += [(per, chain, keep) for (per, chain, _, _), keep in zip(rest, keeps) if keep < len(chain)]
                break
    dropped = np.zeros(n, dtype=bool)
    for per, chain, keep in plan:
        start = chain[0][0]
        total = sum(key[1] for key in chain)
        size = -(-(-(-total // keep)) // 64) * 64  # ceil(total / keep), up to a multiple of 64
        for i, key in enumerate(chain):
            if i < keep and i * size < total:
                kv_o[runs[key]] = start + i * size
                kv_l[runs[key]] = min(size, total - i * size)
            else:
                dropped[runs[key]] = True
    if not dropped.any():
        return unchanged()
    entries = np.asarray(req_entries, dtype=np.int64)
    lens = np.asarray(req_lens, dtype=np.int64)
    offs = np.asarray(req_offs, dtype=np.int64)
    total = int(lens.sum())
    if not np.array_equal(offs, np.concatenate([[0], np.cumsum(lens)[:-1]])):
        raise ValueError("the per-request lists must lie back to back in request order")
    row_dropped = np.zeros(len(q_ent), dtype=bool)
    for v in np.nonzero(dropped)[0]:
        row_dropped[q_o[v]: q_o[v] + q_l[v]] = True
    listed = entries[:total]
    keep = ~row_dropped[listed]
    owner = np.repeat(np.arange(len(lens)), lens)
    new_lens = np.bincount(owner[keep], minlength=len(lens))
    new_offs = np.concatenate([[0], np.cumsum(new_lens)[:-1]])
    new_entries = np.concatenate([listed[keep], np.full(32, -1, dtype=np.int64)])
    kept = ~dropped
    n0 = int(kept[:count0].sum())
    out = (kv_o[kept].astype(np.int32), kv_l[kept].astype(np.int32), q_o[kept].astype(np.int32), q_l[kept].astype(np.int32),
           new_entries.astype(np.int32), new_offs.astype(np.int32), new_lens.astype(np.int32),
           [n0, int(kept.sum()) - n0], [0, n0])
    if return_order:
        where = np.full(n, -1, dtype=np.int64)
        where[kept] = np.arange(int(kept.sum()))
        out = (*out, where)
    return out


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
    launch_order=True,
    buffers=None,
):
    """Drop-in for kernel_bench/fasttree.py:99-296: plan on the host, then place the nine
    int32 index arrays and the two fp32 partial-result buffers on ``device``.

    Returns ``((vnode_to_kv_entries, vnode_to_kv_offs, vnode_to_kv_lens,
    vnode_to_q_entries, vnode_to_q_offs, vnode_to_q_lens, req_to_vnode_entries,
    req_to_vnode_offs, req_to_vnode_lens, mid_o, mid_lse, phase_node_nums,
    phase_node_offsets), node_assignments)``.  The keyword-only arguments do not exist
    in the reference: ``device`` defaults to the reference's hard-wired "cuda";
    ``kv_slot_map`` is described in :func:`fasttree_plan`; ``launch_order`` arranges the vnodes
    for the kernels (:func:`join_kv_chunks`, then :func:`vnodes_in_launch_order`) instead of
    leaving them in the reference's order; with ``buffers`` (a :class:`PlanBuffers`) nothing is allocated on the device: the
    arrays are written into its buffers and the returned tensors are their leading parts.
    """
    import torch

    plan = fasttree_plan(
        tree_info, KV_ptrs, batch_size, num_kv_heads,
        KV_SPLIT_SIZES, para_threshs1, para_threshs2, params, kv_slot_map=kv_slot_map,
    )

    names = iter(("vnode_to_kv_entries", "vnode_to_kv_offs", "vnode_to_kv_lens", "vnode_to_q_entries", "vnode_to_q_offs",
                  "vnode_to_q_lens", "req_to_vnode_entries", "req_to_vnode_offs", "req_to_vnode_lens"))

    def put(values):
        name = next(names)  # (the nine arrays are placed in this order below)
        if buffers is not None:
            return buffers.fill(name, values)
        host = torch.from_numpy(np.ascontiguousarray(np.asarray(values, dtype=np.int32)))
        return host.to(device)

    rows = plan.num_rows
    vnodes = (plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
              plan.phase_node_nums, plan.phase_node_offsets)
    per_request = (plan.req_to_vnode_entries, plan.req_to_vnode_offs, plan.req_to_vnode_lens)
    if launch_order:
        group = max(1, num_qo_heads // num_kv_heads)
        joined = join_kv_chunks(*vnodes[:4], plan.vnode_to_q_entries, *per_request, *vnodes[4:], group, num_kv_heads)
        vnodes, per_request = (*joined[:4], *joined[7:]), joined[4:7]
        vnodes = vnodes_in_launch_order(*vnodes, group, num_kv_heads, q_tile=params.TSQs[0])
    if buffers is not None:
        if rows > buffers.mid_o.shape[0] or buffers.mid_o.shape[1:] != (num_qo_heads, head_dim):
            raise ValueError(f"the scratch of the buffers ({tuple(buffers.mid_o.shape)}) does not hold "
                             f"{rows} rows of {num_qo_heads} x {head_dim}")
        mid_o, mid_lse = buffers.mid_o[:rows], buffers.mid_lse[:rows]
    else:
        mid_o = torch.empty((rows, num_qo_heads, head_dim), dtype=torch.float32, device=device)
        mid_lse = torch.empty((rows, num_qo_heads), dtype=torch.float32, device=device)
    aux = (
        put(plan.vnode_to_kv_entries),
        put(vnodes[0]),
        put(vnodes[1]),
        put(plan.vnode_to_q_entries),
        put(vnodes[2]),
        put(vnodes[3]),
        put(per_request[0]),
        put(per_request[1]),
        put(per_request[2]),
        mid_o,
        mid_lse,
        list(vnodes[4]),
        list(vnodes[5]),
    )
    return aux, plan.node_assignments
