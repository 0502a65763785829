"""SGLang v0.2.13 decode hook on top of the HIP kernels.

Mirrors the reference plugin ``fasttree_sglang_plugin_v0_2_13``:

* ``FastTreeMetadata``          -- metadata.py:5-66 (pre-allocated device buffers, same
  constructor arguments, defaults and attribute names);
* ``decode_forward_fasttree``   -- plugin.py:15-51 (the body bound to
  ``RadixAttention.decode_forward``);
* ``prepare_for_fasttree_meta`` / ``prepare_for_fasttree_step`` -- schedule.py:12-283 (the
  per-batch planner over the radix cache and the in-place ``kv_len += 1`` between decode steps);
* ``load_fasttree_plugin``      -- plugin.py:234-238.

Nothing here imports sglang at module import time.  The hook and the planner only use the
attributes of the objects they are handed (duck typing), so they run against SGLang's own
``RadixAttention`` / ``InputMetadata`` / ``ScheduleBatch`` / ``TreeNode`` and against any object
with the same fields.
"""

from __future__ import annotations

from collections import defaultdict, deque
from types import MethodType
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch


class FastTreeMetadata:
    """Planner hyper-parameters plus the device buffers one decode step reads (metadata.py:5-66).

    Buffers are allocated once at their maxima; a plan fills prefixes of them.  The defaults are
    the reference's, including ``para_threshs1=(132, 132)`` / ``para_threshs2=(132, 528)``
    (132 = compute units of an H100; an MI355X has 256).
    """

    def __init__(
        self,
        num_qo_heads: int,
        num_kv_heads: int,
        head_dim: int,
        device="cuda",
        alpha: float = 0.6,
        beta: float = 0.3,
        gamma: float = 0.1,
        TSQs: Optional[Tuple[int, int]] = None,
        TSKs: Tuple[int, int] = (32, 32),
        kv_split_sizes: Tuple[int, int] = (1024, 128),
        para_threshs1: Tuple[int, int] = (132, 132),
        para_threshs2: Tuple[int, int] = (132, 528),
        max_vnodes: int = 16384,
        max_vnode_to_q_entries: int = 81920,
        max_batch_size: int = 8192,
        fused_store: bool = False,
        launch_order: bool = True,
        fix_enumerate: bool = False,
    ):
        self.num_qo_heads = num_qo_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.kv_group_num = num_qo_heads // num_kv_heads
        self.device = device
        self.alpha, self.beta, self.gamma = alpha, beta, gamma
        self.TSQs = TSQs if TSQs is not None else (64 // self.kv_group_num, 16 // self.kv_group_num)
        self.TSKs = TSKs
        self.kv_split_sizes = kv_split_sizes
        self.para_threshs1 = para_threshs1
        self.para_threshs2 = para_threshs2
        #: not in the reference: the hook writes the step's K/V rows with this library's single
        #: launch instead of calling the layer's ``store_kv_cache``
        self.fused_store = fused_store
        #: not in the reference: the vnode lists are arranged as block programs for the kernels
        #: (launch_schedule.block_programs) instead of left in the reference's order
        self.launch_order = launch_order
        #: not in the reference: evaluate the cost model and merge nodes into their children where
        #: it says so (what schedule.py:87-118 sets out to do; as shipped its loop over
        #: ``enumerate(node.children.values())`` never finds a child and nothing is ever merged).
        #: Off by default = the shipped behaviour.
        self.fix_enumerate = fix_enumerate

        def ints(n):
            return torch.empty(n, dtype=torch.int32, device=device)

        self.vnode_to_q_entries = ints(max_vnode_to_q_entries)
        self.vnode_to_q_offs = ints(max_vnodes)
        self.vnode_to_q_lens = ints(max_vnodes)
        self.vnode_to_kv_offs = ints(max_vnodes)
        self.vnode_to_kv_lens = ints(max_vnodes)
        self.req_to_vnode_entries = ints(max_vnode_to_q_entries)
        self.req_to_vnode_offs = ints(max_batch_size)
        self.req_to_vnode_lens = ints(max_batch_size)
        self.mid_o = torch.empty((max_vnode_to_q_entries, num_qo_heads, head_dim), dtype=torch.float32, device=device)
        self.mid_lse = torch.empty((max_vnode_to_q_entries, num_qo_heads), dtype=torch.float32, device=device)
        #: not in the reference: the block programs of a launch-order plan (four entries each)
        self.prog_table = ints(4 * max_vnodes)
        #: not in the reference: a launch-order plan's record per request for the merge launch
        self.req_table = ints(16 * max_batch_size)

        self.phase_node_nums: Optional[Sequence[int]] = None
        self.phase_node_offsets: Optional[Sequence[int]] = None
        self.phase_q_tile_sizes: Optional[Sequence[int]] = None
        self.phase_kv_tile_sizes: Optional[Sequence[int]] = None
        self.req_last_vnodes: Optional[List[int]] = None

        print("FastTreeMetadata initialized")


# ---------------------------------------------------------------------------------------
# The hook body
# ---------------------------------------------------------------------------------------
def decode_forward_fasttree(self, q, k, v, input_metadata):
    """``RadixAttention.decode_forward`` replacement (plugin.py:15-51).

    Stores the step's K/V rows through the layer's own ``store_kv_cache`` (or, with
    ``FastTreeMetadata(fused_store=True)``, with one launch of this library for both pools), then
    runs the tree decode with the pool buffers, ``req_to_token`` as the flat KV-index array and
    the metadata bound to ``input_metadata.fasttree``.  The output shape for ``qk_head_dim != v_head_dim``
    follows the reference literally (plugin.py:22-23).
    """
    from .decode import fasttree_decode, store_kv_cache

    if self.qk_head_dim != self.v_head_dim:
        o = q.new_empty((q.shape[-1], self.tp_q_head_num * self.v_head_dim))
    else:
        o = torch.empty_like(q)
    meta = input_metadata.fasttree
    if getattr(meta, "fused_store", False):
        store_kv_cache(k, v, input_metadata.out_cache_loc,
                       input_metadata.token_to_kv_pool.get_key_buffer(self.layer_id),
                       input_metadata.token_to_kv_pool.get_value_buffer(self.layer_id))
    else:
        self.store_kv_cache(k, v, input_metadata)

    fasttree_decode(
        q.view(-1, self.tp_q_head_num, self.qk_head_dim),
        input_metadata.token_to_kv_pool.get_key_buffer(self.layer_id),
        input_metadata.token_to_kv_pool.get_value_buffer(self.layer_id),
        o.view(-1, self.tp_q_head_num, self.v_head_dim),
        input_metadata.req_to_token_pool.req_to_token,
        meta.vnode_to_kv_offs, meta.vnode_to_kv_lens,
        meta.vnode_to_q_entries, meta.vnode_to_q_offs, meta.vnode_to_q_lens,
        meta.req_to_vnode_entries, meta.req_to_vnode_offs, meta.req_to_vnode_lens,
        meta.mid_o, meta.mid_lse,
        meta.phase_node_nums, meta.phase_node_offsets,
        meta.phase_q_tile_sizes, meta.phase_kv_tile_sizes,
        sm_scale=self.scaling,
        logit_cap=self.logit_cap,
    )
    return o


# ---------------------------------------------------------------------------------------
# The per-batch planner over the radix cache
# ---------------------------------------------------------------------------------------
def _requests_per_radix_node(batch) -> Dict[object, List[int]]:
    """Walks every request's token sequence (prompt, then generated tokens) down the radix tree
    and lists, per node reached, the batch positions of the requests (schedule.py:18-35)."""
    reqs_of = defaultdict(list)
    for rid, req in enumerate(batch.reqs):
        tokens_in, tokens_out = req.origin_input_ids, req.output_ids
        total = len(tokens_in) + len(tokens_out)
        node, pos = batch.tree_cache.root_node, 0
        while pos < total:
            token = tokens_in[pos] if pos < len(tokens_in) else tokens_out[pos - len(tokens_in)]
            child = node.children.get(token)
            if not child:
                break
            reqs_of[child].append(rid)
            node = child
            pos += len(child.key)
    return reqs_of


def prepare_for_fasttree_meta(batch, fasttree_metadata: FastTreeMetadata):
    """Plans one decode batch (schedule.py:12-277) and binds the metadata to it.

    As shipped, the reference's merge loop never takes a decision: it iterates
    ``enumerate(node.children.values())`` (schedule.py:96), whose tuples are never keys of the
    request map, so every radix node keeps its own vnodes (assignment 0 everywhere).  That is
    the behaviour restated here; the cost model is therefore not evaluated.  Other literal
    traits kept: the kv-split "reduction" of the first adaptation pass assigns a value to
    itself (schedule.py:126), the second pass sets the KV tile sizes from the already replaced
    query tile list (schedule.py:137-141), and parallelism counts KV *tiles*, not splits
    (schedule.py:113).
    """
    meta = fasttree_metadata
    root = batch.tree_cache.root_node
    reqs_of = _requests_per_radix_node(batch)

    # live nodes in BFS order with the offset of their first token along the path
    order, token_offset, parent_of = [], [], []
    todo = deque([(root, 0, -1)])
    while todo:
        node, off, up = todo.popleft()
        order.append(node)
        token_offset.append(off)
        parent_of.append(up)
        for child in node.children.values():
            if child in reqs_of:
                todo.append((child, off + len(node.value), len(order) - 1))

    n_reqs = [len(reqs_of[node]) if node in reqs_of else 0 for node in order]
    seqlens = [len(node.value) for node in order]
    merge = bool(getattr(meta, "fix_enumerate", False))
    own_lens, all_reqs = list(seqlens), [list(reqs_of[node]) if node in reqs_of else [] for node in order]
    members_of, start_of = None, list(token_offset)

    def decide(q_tiles, kv_tiles):
        """The cost model's decisions for the current tile sizes: per node the requests its own
        vnodes serve, the tokens they attend (its own and those of the ancestors merged into
        it) and where that run starts along the path."""
        from .kv_tree import KVTreeNode
        from .planner import FastTreeParams, _run_chain, _tree_heuristic

        params = FastTreeParams()
        params.set_values(meta.alpha, meta.beta, meta.gamma)
        params.set_q_tile_sizes(list(q_tiles)); params.set_kv_tile_sizes(list(kv_tiles))
        params.set_kv_group_num(meta.kv_group_num)
        info = []
        for i, up in enumerate(parent_of):
            n = KVTreeNode(parent=up, id=i, seqlen=own_lens[i])
            n.requests = all_reqs[i] if i else list(range(len(batch.reqs)))
            info.append(n)
        for up in parent_of[1:]:
            info[up].num_children += 1
        assignment = _tree_heuristic(info, params)
        children = [[] for _ in order]
        for c, up in enumerate(parent_of):
            if up >= 0:
                children[up].append(c)
        served = []
        for i in range(len(order)):
            gone = set(r for c in children[i] if assignment[c] == 1 for r in all_reqs[c])
            listed = [r for c in children[i] if assignment[c] == 0 for r in all_reqs[c]]  # child by child, as the reference lists them
            seen = set(listed) | gone
            listed += [r for r in all_reqs[i] if r not in seen]             # requests whose prompt ends at this node
            served.append(listed if i else [])
        lens, starts = [], []
        for i in range(len(order)):
            chain, total = _run_chain(info, assignment, i) if i else ([0], 0)
            lens.append(total)
            starts.append(token_offset[chain[0]])
        return served, lens, starts

    q_tiles = meta.TSQs
    kv_tiles = meta.TSKs
    kv_splits = [meta.kv_split_sizes[0], meta.kv_split_sizes[0]]

    def parallelism():
        p = [0, 0]
        for nq, length in zip(n_reqs, seqlens):
            if nq > 0:
                phase = 0 if nq > q_tiles[1] else 1
                p[phase] += ((nq - 1) // q_tiles[phase] + 1) * ((length - 1) // kv_tiles[phase] + 1)
        return [x * meta.num_kv_heads for x in p]

    for it in range(3):
        if merge:
            members_of, seqlens, start_of = decide(q_tiles, kv_tiles)
            n_reqs = [len(m) for m in members_of]
        p = parallelism()
        if it == 0:
            low = [ph for ph in range(2) if 0 < p[ph] < meta.para_threshs1[ph]]
            for ph in low:
                kv_splits[ph] = kv_splits[1]
            if not low:
                break
        elif it == 1:
            if 0 < p[0] < meta.para_threshs2[0]:
                q_tiles = [q_tiles[1], q_tiles[1]]
                kv_tiles = [q_tiles[1], q_tiles[1]]
            elif 0 < p[1] < meta.para_threshs2[1]:
                q_tiles = [q_tiles[0], q_tiles[0]]
                kv_tiles = [q_tiles[0], q_tiles[0]]
            else:
                break
    meta.phase_q_tile_sizes = q_tiles
    meta.phase_kv_tile_sizes = kv_tiles

    kv_offs, kv_lens, q_entries, q_offs, q_lens = [], [], [], [], []
    rows = batch.req_pool_indices.cpu()
    stride = batch.req_to_token_pool.req_to_token.stride(0)

    def emit(kv_start, length, members, q_tile, kv_split, n_q):
        # one copy of the member list per KV split, cut into query tiles
        for kv0 in range(0, length, kv_split):
            q0 = len(q_entries)
            q_entries.extend(members)
            for s in range(0, n_q, q_tile):
                kv_offs.append(kv_start + kv0)
                kv_lens.append(min(kv0 + kv_split, length) - kv0)
                q_offs.append(q0 + s)
                q_lens.append(min(s + q_tile, n_q) - s)

    if merge:
        members_of, seqlens, start_of = decide(q_tiles, kv_tiles)   # (for the tile sizes the passes settled on)
        n_reqs = [len(m) for m in members_of]
    for i, (node, nq, length, off) in enumerate(zip(order, n_reqs, seqlens, start_of)):
        if nq == 0:
            continue
        # the members are listed child by child where the node has live children (all of them
        # keep assignment 0), else from the node itself; the KV is read through the row of the
        # first member
        if merge:
            members = members_of[i]
        else:
            groups = [c for c in node.children.values() if c in reqs_of] or [node]
            members = [r for grp in groups for r in reqs_of[grp]]
        phase = 0 if nq > q_tiles[1] else 1
        emit(stride * int(rows[members[0]]) + off, length, members, q_tiles[phase], kv_splits[phase], nq)

    # generated tokens: one chain of single-request vnodes per request, after the tree's
    last = [0] * len(batch.reqs)
    for rid, req in enumerate(batch.reqs):
        prefix = len(req.origin_input_ids)
        emit(stride * int(rows[rid]) + prefix, len(req.output_ids) + 1, [rid], 1, kv_splits[1], 1)
        last[rid] = len(kv_lens) - 1  # unchanged by the reordering below
    meta.req_last_vnodes = last

    per_req = [[] for _ in batch.reqs]
    for row, r in enumerate(q_entries):
        per_req[r].append(row)
    req_offs, req_lens, acc = [], [], 0
    for lst in per_req:
        req_offs.append(acc)
        req_lens.append(len(lst))
        acc += len(lst)
    req_entries = [row for lst in per_req for row in lst]

    above = [i for i, n in enumerate(q_lens) if n > q_tiles[1]]
    below = [i for i, n in enumerate(q_lens) if n <= q_tiles[1]]
    perm = above + below
    meta.phase_node_nums = [len(above), len(below)]
    meta.phase_node_offsets = [0, len(above)]
    lists = [[x[i] for i in perm] for x in (kv_offs, kv_lens, q_offs, q_lens)]
    meta.prog_table_len = 0
    if getattr(meta, "launch_order", False):
        from . import launch_schedule
        from .launch_schedule import LaunchPhases, block_programs

        # the same computation as block programs: long shared runs (a system prompt
        # under a large batch) cut where the machine is full instead of at the KV split
        tail_ends = [lists[0][v] + lists[1][v] for v in meta.req_last_vnodes]
        from .launch_schedule import compute_units
        sched = block_programs(*lists, q_entries, len(batch.reqs), meta.kv_group_num, meta.num_kv_heads,
                               head_dim=meta.head_dim, num_cus=compute_units(meta.device))
        lists = [sched.kv_offs, sched.kv_lens, sched.q_offs, sched.q_lens]      # (int32 arrays, uploaded as they are)
        q_entries = sched.q_entries
        req_entries = sched.req_entries[: sched.num_rows]
        req_offs, req_lens = sched.req_offs, sched.req_lens
        # a request's last vnode is the single-request vnode that ends where its tokens end
        # (narrow vnodes keep the planner's chunks, so there is exactly one)
        single = np.flatnonzero(sched.q_lens == 1)
        ends = (sched.kv_offs[single].astype(np.int64) + sched.kv_lens[single]).tolist()
        owner = sched.q_entries[sched.q_offs[single]].tolist()
        ends_of = dict(zip(zip(ends, owner), single.tolist()))
        meta.req_last_vnodes = [ends_of[(end, rid)] for rid, end in enumerate(tail_ends)]
        nums = LaunchPhases(sched.phase_node_nums)
        if sched.num_programs > 0:
            table = sched.prog_table.reshape(-1)
            if table.size > meta.prog_table.numel():
                raise ValueError(f"{sched.num_programs} block programs do not fit the {meta.prog_table.numel() // 4} "
                                 "that max_vnodes allows")
            src = torch.from_numpy(np.ascontiguousarray(table))
            meta.prog_table[: src.numel()].copy_(src, non_blocking=True)
            nums.prog_table = meta.prog_table[: src.numel()]
            nums.num_programs = sched.num_programs
            nums.narrow_in_programs = sched.narrow_in_programs
        if sched.num_programs > 0 and launch_schedule.USE_REQUEST_RECORDS and len(req_offs) * 16 <= meta.req_table.numel():
            src = torch.from_numpy(launch_schedule.request_records(req_entries, req_offs, req_lens).reshape(-1))
            meta.req_table[: src.numel()].copy_(src, non_blocking=True)
            nums.req_table = meta.req_table[: src.numel()]
        meta.phase_node_nums, meta.phase_node_offsets = nums, list(sched.phase_node_offsets)

    def upload(dst, values):
        if isinstance(values, np.ndarray):
            src = torch.from_numpy(np.ascontiguousarray(values, dtype=np.int32))
        else:
            src = torch.tensor(values, device="cpu", dtype=torch.int32)
        dst[: src.numel()].copy_(src, non_blocking=True)

    upload(meta.vnode_to_q_entries, q_entries)
    upload(meta.vnode_to_kv_offs, lists[0])
    upload(meta.vnode_to_kv_lens, lists[1])
    upload(meta.vnode_to_q_offs, lists[2])
    upload(meta.vnode_to_q_lens, lists[3])
    upload(meta.req_to_vnode_entries, req_entries)
    upload(meta.req_to_vnode_offs, req_offs)
    upload(meta.req_to_vnode_lens, req_lens)

    batch.fasttree_metadata = meta


def prepare_for_fasttree_step(batch, fasttree_metadata: FastTreeMetadata):
    """Between two decode steps of an unchanged batch every request has one more token: its
    last vnode grows by one, on the device (schedule.py:280-283)."""
    bs = len(batch.reqs)
    one = torch.ones(bs, device=fasttree_metadata.device, dtype=torch.int32)
    fasttree_metadata.vnode_to_kv_lens[fasttree_metadata.req_last_vnodes] += one


# ---------------------------------------------------------------------------------------
# Loader
# ---------------------------------------------------------------------------------------
def annotate_function(owner, func_name):
    """Replaces ``owner.func_name`` by a version that runs inside a named profiler range with a
    device synchronisation on either side, so that a trace shows the step's host and device time
    under that name (plugin.py:70-83; the reference uses the ``nvtx`` package, this uses the
    ranges torch exposes, which are roctx ranges on ROCm)."""
    original = getattr(owner, func_name)

    def annotated(*args, **kwargs):
        if torch.cuda.is_available():
            torch.cuda.synchronize()
        torch.cuda.nvtx.range_push(func_name)
        try:
            return original(*args, **kwargs)
        finally:
            if torch.cuda.is_available():
                torch.cuda.synchronize()
            torch.cuda.nvtx.range_pop()

    annotated.__wrapped__ = original
    setattr(owner, func_name, annotated)


def same_requests(planned_for, reqs) -> bool:
    """Whether ``reqs`` are, one by one, the very objects of ``planned_for`` (a tuple kept from
    the batch the plan was made for, or None).  The tuple holds the request objects themselves,
    so none of them can have been freed and its address given to a new request in between, which
    a comparison of ``id()`` values could not rule out (plugin.py:213-231 re-plans whenever the
    reference's batch object changes)."""
    return (planned_for is not None and len(planned_for) == len(reqs)
            and all(a is b for a, b in zip(planned_for, reqs)))


def plan_or_step(server, batch, replan_every, plan=None, step=None):
    """What the patched ``forward_decode_batch`` does before every decode forward: a new plan when
    the batch does not hold the very requests the last plan was made for, or when that plan has
    served ``replan_every`` forwards; the in-place ``+1`` step otherwise.  The reference plans at
    the top of every ``forward_step`` and steps between the ``num_continue_decode_steps``
    forwards of that step (plugin.py:108-131); ``replan_every`` is that number.  ``server`` keeps
    ``_fasttree_planned_for`` (a tuple of the request objects) and ``_fasttree_forwards``."""
    plan = plan or prepare_for_fasttree_meta
    step = step or prepare_for_fasttree_step
    served = getattr(server, "_fasttree_forwards", 0)
    if same_requests(getattr(server, "_fasttree_planned_for", None), batch.reqs) and served < replan_every:
        step(batch, server.fasttree_metadata)
        server._fasttree_forwards = served + 1
        return "step"
    plan(batch, server.fasttree_metadata)
    server._fasttree_planned_for = tuple(batch.reqs)
    server._fasttree_forwards = 1
    return "plan"


def load_fasttree_plugin(enable_fasttree=True, annotate_breakdown=False):
    """Installs the hook into SGLang v0.2.13 (plugin.py:234-238).

    With the reference's plugin package importable, its loader is used unchanged with the
    kernel entry point, the metadata class and the planner swapped for the ones in this module.
    Without it, the three patches are applied here: ``RadixAttention.decode_forward``,
    ``InputMetadata.from_schedule_batch`` (carries ``batch.fasttree_metadata``), and
    ``ModelTpServer`` (metadata creation; a fresh plan when the batch changed, the ``+1`` step
    otherwise, before every decode forward).  ``annotate_breakdown`` wraps the prefill and decode
    forwards and the two planner entry points in named profiler ranges (plugin.py:68-89).
    Raises ImportError when sglang is not installed.
    """
    if not enable_fasttree and not annotate_breakdown:
        print("[Warning] FastTree plugin is not enabled")
        return
    import sys

    from .decode import fasttree_decode

    this = sys.modules[__name__]
    try:
        import fasttree_sglang_plugin_v0_2_13.plugin as ref_plugin
        import fasttree_sglang_plugin_v0_2_13.schedule as ref_schedule
    except ImportError:
        ref_plugin = None
    if ref_plugin is not None:
        ref_plugin.fasttree_decode = fasttree_decode
        ref_plugin.FastTreeMetadata = FastTreeMetadata
        ref_schedule.prepare_for_fasttree_meta = this.prepare_for_fasttree_meta
        ref_schedule.prepare_for_fasttree_step = this.prepare_for_fasttree_step
        return ref_plugin.load_fasttree_plugin(enable_fasttree, annotate_breakdown)

    from sglang.srt.layers.radix_attention import RadixAttention
    from sglang.srt.managers.tp_worker import ModelTpServer
    from sglang.srt.model_executor.forward_batch_info import InputMetadata

    if annotate_breakdown:
        annotate_function(ModelTpServer, "forward_prefill_batch")
        annotate_function(ModelTpServer, "forward_decode_batch")
        if enable_fasttree:
            annotate_function(this, "prepare_for_fasttree_meta")
            annotate_function(this, "prepare_for_fasttree_step")
    if not enable_fasttree:
        return

    radix_init = RadixAttention.__init__

    def radix_init_with_hook(self, *args, **kwargs):
        radix_init(self, *args, **kwargs)
        self.decode_forward = MethodType(decode_forward_fasttree, self)

    RadixAttention.__init__ = radix_init_with_hook

    meta_from_batch = InputMetadata.from_schedule_batch.__func__

    def meta_from_batch_with_plan(cls, model_runner, batch, forward_mode):
        ret = meta_from_batch(cls, model_runner, batch, forward_mode)
        ret.fasttree = getattr(batch, "fasttree_metadata", None)
        return ret

    InputMetadata.from_schedule_batch = classmethod(meta_from_batch_with_plan)

    server_init = ModelTpServer.__init__

    def server_init_with_metadata(self, gpu_id, tp_rank, server_args, nccl_port, model_overide_args):
        server_args.disable_cuda_graph = True  # plugin.py:209-211
        server_init(self, gpu_id, tp_rank, server_args, nccl_port, model_overide_args)
        self.fasttree_metadata = FastTreeMetadata(
            self.model_config.num_attention_heads, self.model_config.num_key_value_heads,
            self.model_config.head_dim, torch.device("cuda", self.gpu_id))
        self._fasttree_planned_for = None
        self._fasttree_forwards = 0

    ModelTpServer.__init__ = server_init_with_metadata

    decode_batch = ModelTpServer.forward_decode_batch

    try:
        from sglang.global_config import global_config
        replan_every = int(global_config.num_continue_decode_steps)
    except Exception:
        replan_every = 10

    def decode_batch_with_plan(self, batch):
        plan_or_step(self, batch, replan_every, this.prepare_for_fasttree_meta, this.prepare_for_fasttree_step)
        return decode_batch(self, batch)

    ModelTpServer.forward_decode_batch = decode_batch_with_plan
