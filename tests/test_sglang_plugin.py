"""The SGLang hook mirror: planner over a radix cache (CPU) and the hook body (GPU).

The reference's plugin imports sglang at module level (schedule.py:6-7, plugin.py:2), which is
not installed here, so no golden vectors exist for this planner: the first test is a
known-answer case derived by hand from schedule.py:12-277, the others check the invariants any
correct plan has (every token of every request is covered by exactly one of the request's
scratch rows).  Parity of the array *order* beyond the hand case is unpinned.
"""
import math
import random

import pytest
import torch

from fasttree_hip.sglang_plugin import (FastTreeMetadata, decode_forward_fasttree, prepare_for_fasttree_meta,
                                        prepare_for_fasttree_step)


# ---- stand-ins with the fields of SGLang's TreeNode / Req / ScheduleBatch / pools
class Node:
    def __init__(self, key=(), value=()):
        self.key, self.value, self.children = list(key), list(value), {}


class Req:
    def __init__(self, origin_input_ids, output_ids):
        self.origin_input_ids, self.output_ids = list(origin_input_ids), list(output_ids)


class Obj:
    def __init__(self, **kw):
        self.__dict__.update(kw)


def insert(root, tokens, slots):
    """Radix insert without node splitting: callers insert shared prefixes first."""
    node, pos = root, 0
    while pos < len(tokens):
        child = node.children.get(tokens[pos])
        if child is None:
            child = Node(tokens[pos:], slots[pos:])
            node.children[tokens[pos]] = child
            return
        assert tokens[pos:pos + len(child.key)] == child.key
        node, pos = child, pos + len(child.key)


def make_batch(prompts, outputs, shared_prefixes, device="cpu", max_ctx=64, row_of=None):
    """prompts[r]: token ids; shared_prefixes: token lists inserted first as their own nodes.
    Pool slots are handed out so that shared prefixes own the same slots in every row."""
    root = Node()
    slot_of_prefix = {}
    next_slot = [1]

    def slots_for(tokens):
        out = []
        for i in range(len(tokens)):
            key = tuple(tokens[: i + 1])
            if key not in slot_of_prefix:
                slot_of_prefix[key] = next_slot[0]
                next_slot[0] += 1
            out.append(slot_of_prefix[key])
        return out

    for pre in shared_prefixes:
        insert(root, pre, slots_for(pre))
    for p in prompts:
        insert(root, p, slots_for(p))
    n = len(prompts)
    row_of = row_of or list(range(n))
    req_to_token = torch.zeros((max(row_of) + 1, max_ctx), dtype=torch.int32)
    for r, (p, out) in enumerate(zip(prompts, outputs)):
        sl = slots_for(p)
        gen = list(range(next_slot[0], next_slot[0] + len(out) + 1))  # generated tokens + the one being decoded
        next_slot[0] += len(out) + 1
        req_to_token[row_of[r], : len(sl) + len(gen)] = torch.tensor(sl + gen, dtype=torch.int32)
    batch = Obj(reqs=[Req(p, o) for p, o in zip(prompts, outputs)], tree_cache=Obj(root_node=root),
                req_pool_indices=torch.tensor(row_of, dtype=torch.int64, device=device),
                req_to_token_pool=Obj(req_to_token=req_to_token.to(device)))
    return batch, next_slot[0]


def plan_lists(meta, batch):
    nv = sum(meta.phase_node_nums)
    rows = int(meta.req_to_vnode_offs[len(batch.reqs) - 1] + meta.req_to_vnode_lens[len(batch.reqs) - 1])
    # (rows of chunks the launch order dropped stay in the scratch, unlisted: the rows that are in use may end later)
    used = max(rows, int((meta.vnode_to_q_offs[:nv] + meta.vnode_to_q_lens[:nv]).max()))
    return dict(kv_offs=meta.vnode_to_kv_offs[:nv].tolist(), kv_lens=meta.vnode_to_kv_lens[:nv].tolist(),
                q_offs=meta.vnode_to_q_offs[:nv].tolist(), q_lens=meta.vnode_to_q_lens[:nv].tolist(),
                q_entries=meta.vnode_to_q_entries[:used].tolist(), req_entries=meta.req_to_vnode_entries[:rows].tolist(),
                req_offs=meta.req_to_vnode_offs[: len(batch.reqs)].tolist(),
                req_lens=meta.req_to_vnode_lens[: len(batch.reqs)].tolist())


def small_meta(device="cpu", hq=32, hkv=8, d=128, **kw):
    return FastTreeMetadata(hq, hkv, d, device=device, max_vnodes=4096, max_vnode_to_q_entries=8192,
                            max_batch_size=512, **kw)


def test_metadata_defaults_follow_the_reference():
    m = small_meta()
    assert m.kv_group_num == 4 and m.TSQs == (16, 4) and m.TSKs == (32, 32)
    assert m.kv_split_sizes == (1024, 128) and m.para_threshs1 == (132, 132) and m.para_threshs2 == (132, 528)
    assert (m.alpha, m.beta, m.gamma) == (0.6, 0.3, 0.1)
    assert m.mid_o.shape == (8192, 32, 128) and m.mid_o.dtype == torch.float32
    assert m.mid_lse.shape == (8192, 32)
    for t in (m.vnode_to_q_entries, m.vnode_to_q_offs, m.vnode_to_kv_lens, m.req_to_vnode_entries, m.req_to_vnode_offs):
        assert t.dtype == torch.int32
    assert FastTreeMetadata(64, 8, 128, device="cpu", max_vnodes=8, max_vnode_to_q_entries=8, max_batch_size=8).TSQs == (8, 2)


def test_hand_derived_plan():
    # radix tree: A=[1,2,3,4] -> B=[5,6] (request 0), C=[7,8,9] (requests 1, 2)
    prompts = [[1, 2, 3, 4, 5, 6], [1, 2, 3, 4, 7, 8, 9], [1, 2, 3, 4, 7, 8, 9]]
    outputs = [[10, 11], [12], []]
    batch, _ = make_batch(prompts, outputs, shared_prefixes=[[1, 2, 3, 4]], row_of=[2, 0, 5])
    meta = small_meta(launch_order=False)  # the reference's own order
    prepare_for_fasttree_meta(batch, meta)
    s = 64  # row stride of req_to_token
    # parallelism [0, 24] < thresholds: pass 0 leaves the splits, pass 1 takes its second branch
    assert list(meta.phase_q_tile_sizes) == [16, 16] and list(meta.phase_kv_tile_sizes) == [16, 16]
    assert list(meta.phase_node_nums) == [0, 6] and list(meta.phase_node_offsets) == [0, 0]
    got = plan_lists(meta, batch)
    assert got["kv_offs"] == [2 * s + 0, 2 * s + 4, 0 * s + 4, 2 * s + 6, 0 * s + 7, 5 * s + 7]
    assert got["kv_lens"] == [4, 2, 3, 3, 2, 1]
    assert got["q_offs"] == [0, 3, 4, 6, 7, 8]
    assert got["q_lens"] == [3, 1, 2, 1, 1, 1]
    assert got["q_entries"] == [0, 1, 2, 0, 1, 2, 0, 1, 2]
    assert got["req_entries"] == [0, 3, 6, 1, 4, 7, 2, 5, 8]
    assert got["req_offs"] == [0, 3, 6] and got["req_lens"] == [3, 3, 3]
    assert meta.req_last_vnodes == [3, 4, 5]
    assert batch.fasttree_metadata is meta
    covered = [sorted(x) for x in covered_slots(meta, batch)]
    prepare_for_fasttree_step(batch, meta)
    assert meta.vnode_to_kv_lens[:6].tolist() == [4, 2, 3, 4, 3, 2]

    # launch order (the default): the same vnodes with scratch rows of their own; the tail vnodes are found at their new positions
    meta2 = small_meta()
    prepare_for_fasttree_meta(batch, meta2)
    got2 = plan_lists(meta2, batch)
    vnodes = lambda g: sorted((o, n, tuple(g["q_entries"][qo:qo + ql]))
                              for o, n, qo, ql in zip(g["kv_offs"], g["kv_lens"], g["q_offs"], g["q_lens"]))
    assert vnodes(got2) == vnodes(got) and list(meta2.phase_node_nums) == [0, 6]
    assert [sorted(x) for x in covered_slots(meta2, batch)] == covered
    for r in range(3):
        rows = got2["req_entries"][got2["req_offs"][r]: got2["req_offs"][r] + got2["req_lens"][r]]
        assert len(rows) == 3 and all(got2["q_entries"][x] == r for x in rows)
    for r, v in enumerate(meta2.req_last_vnodes):
        assert got2["kv_offs"][v] == got["kv_offs"][[3, 4, 5][r]] and got2["q_entries"][got2["q_offs"][v]] == r
    prepare_for_fasttree_step(batch, meta2)
    assert sorted(meta2.vnode_to_kv_lens[:6].tolist()) == sorted([4, 2, 3, 4, 3, 2])


def covered_slots(meta, batch):
    """Per request: the multiset of pool slots its scratch rows attend to."""
    flat = batch.req_to_token_pool.req_to_token.reshape(-1).cpu()
    got = plan_lists(meta, batch)
    out = [[] for _ in batch.reqs]
    for kv_off, kv_len, q_off, q_len in zip(got["kv_offs"], got["kv_lens"], got["q_offs"], got["q_lens"]):
        for r in got["q_entries"][q_off:q_off + q_len]:
            out[r] += flat[kv_off:kv_off + kv_len].tolist()
    return out


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_every_token_is_covered_once(seed):
    rng = random.Random(seed)
    n_groups, per_group = rng.randint(1, 4), rng.randint(1, 24)
    system = [rng.randint(1, 10**6) for _ in range(rng.randint(1, 40))]
    prefixes, prompts, outputs = [system], [], []
    for _ in range(n_groups):
        mid = system + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 30))]
        prefixes.append(mid)
        for _ in range(per_group):
            prompts.append(mid + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 12))])
            outputs.append([rng.randint(1, 10**6) for _ in range(rng.randint(0, 5))])
    batch, _ = make_batch(prompts, outputs, prefixes, max_ctx=128)
    meta = small_meta(kv_split_sizes=(16, 8))
    prepare_for_fasttree_meta(batch, meta)
    cov = covered_slots(meta, batch)
    table = batch.req_to_token_pool.req_to_token
    for r, (p, o) in enumerate(zip(prompts, outputs)):
        want = table[r, : len(p) + len(o) + 1].tolist()
        assert sorted(cov[r]) == sorted(want)
    got = plan_lists(meta, batch)
    nv0 = meta.phase_node_nums[0]
    assert all(n > meta.phase_q_tile_sizes[1] for n in got["q_lens"][:nv0])
    assert all(n <= meta.phase_q_tile_sizes[1] for n in got["q_lens"][nv0:])
    for r in range(len(prompts)):
        rows = got["req_entries"][got["req_offs"][r]: got["req_offs"][r] + got["req_lens"][r]]
        assert all(got["q_entries"][i] == r for i in rows) and rows == sorted(rows)


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5])
def test_chunk_joins_keep_the_coverage_and_the_last_vnodes(seed, monkeypatch):
    """The launch order's chunk rule forced on every chain (system prompt, group prefixes,
    prompts and generated tails all longer than the KV split): every request still attends each
    of its tokens once through the rows listed for it, its last vnode is a single-request vnode
    that ends where its tokens end, and the in-place step makes it cover the next token."""
    from fasttree_hip import launch_schedule
    rng = random.Random(100 + seed)
    system = [rng.randint(1, 10**6) for _ in range(rng.randint(20, 60))]
    prefixes, prompts, outputs = [system], [], []
    for _ in range(rng.randint(1, 3)):
        mid = system + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 40))]
        prefixes.append(mid)
        for _ in range(rng.randint(1, 20)):
            prompts.append(mid + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 30))])
            outputs.append([rng.randint(1, 10**6) for _ in range(rng.randint(0, 25))])
    batch, _ = make_batch(prompts, outputs, prefixes, max_ctx=256)
    plain = small_meta(kv_split_sizes=(8, 8), launch_order=False)
    prepare_for_fasttree_meta(batch, plain)
    monkeypatch.setattr(launch_schedule, "MIN_PROGRAM_TILES", 0.0)   # cut every launch anew
    meta = small_meta(kv_split_sizes=(8, 8))
    prepare_for_fasttree_meta(batch, meta)
    assert sum(meta.phase_node_nums) < sum(plain.phase_node_nums), "chunks were joined"
    table = batch.req_to_token_pool.req_to_token
    got = plan_lists(meta, batch)
    flat = table.reshape(-1)
    row_vnode = {}
    for v, (qo, ql) in enumerate(zip(got["q_offs"], got["q_lens"])):
        for i in range(ql):
            assert qo + i not in row_vnode
            row_vnode[qo + i] = v
    listed = set()
    for r, (p, o) in enumerate(zip(prompts, outputs)):
        rows = got["req_entries"][got["req_offs"][r]: got["req_offs"][r] + got["req_lens"][r]]
        assert rows == sorted(set(rows)) and all(got["q_entries"][i] == r for i in rows)
        listed.update(rows)
        seen = []
        for i in rows:
            v = row_vnode[i]
            seen += flat[got["kv_offs"][v]: got["kv_offs"][v] + got["kv_lens"][v]].tolist()
        assert sorted(seen) == sorted(table[r, : len(p) + len(o) + 1].tolist())
        v = meta.req_last_vnodes[r]
        assert got["q_lens"][v] == 1 and got["q_entries"][got["q_offs"][v]] == r
        assert got["kv_offs"][v] + got["kv_lens"][v] == r * table.stride(0) + len(p) + len(o) + 1
    assert listed == set(row_vnode), "no row of a kept vnode is unlisted, no dropped row is listed"
    before = meta.vnode_to_kv_lens[: sum(meta.phase_node_nums)].clone()
    prepare_for_fasttree_step(batch, meta)
    grown = meta.vnode_to_kv_lens[: sum(meta.phase_node_nums)] - before
    assert grown.sum().item() == len(prompts) and all(grown[v].item() == 1 for v in meta.req_last_vnodes)


def test_annotate_function_keeps_results_and_errors():
    """The breakdown wrapper of load_fasttree_plugin(annotate_breakdown=True): same result, same
    exception, the original reachable, the range closed either way."""
    from fasttree_hip.sglang_plugin import annotate_function
    calls = []

    class Owner:
        def work(self, x, y=1):
            calls.append((x, y))
            if x < 0:
                raise ValueError("negative")
            return x + y

    annotate_function(Owner, "work")
    o = Owner()
    assert o.work(2, y=5) == 7 and calls == [(2, 5)]
    with pytest.raises(ValueError):
        o.work(-1)
    assert Owner.work.__wrapped__(o, 3) == 4


# ---- the hook body on the GPU
class FakeLayer:
    def __init__(self, hq, hkv, d, layer_id=0):
        self.tp_q_head_num, self.tp_k_head_num, self.qk_head_dim, self.v_head_dim = hq, hkv, d, d
        self.layer_id, self.scaling, self.logit_cap = layer_id, 1.0 / math.sqrt(d), -1

    def store_kv_cache(self, k, v, input_metadata):
        pool = input_metadata.token_to_kv_pool
        pool.k[self.layer_id][input_metadata.out_cache_loc] = k.view(-1, self.tp_k_head_num, self.qk_head_dim)
        pool.v[self.layer_id][input_metadata.out_cache_loc] = v.view(-1, self.tp_k_head_num, self.v_head_dim)


class FakePool:
    def __init__(self, k, v):
        self.k, self.v = [k], [v]

    def get_key_buffer(self, layer_id):
        return self.k[layer_id]

    def get_value_buffer(self, layer_id):
        return self.v[layer_id]


@pytest.mark.gpu
@pytest.mark.parametrize("joined", [False, True, "reference_order", "merged", "merged_reference_order"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_hook_matches_dense_attention(device, dtype, joined, monkeypatch):
    """`joined`: 32-token KV splits with every launch cut anew into block programs, so that the
    step after it grows tail vnodes that sit at other positions than the planner gave them;
    "reference_order": FastTreeMetadata(launch_order=False), the reference's own lists;
    "merged...": FastTreeMetadata(fix_enumerate=True) with nodes merged into their children."""
    import fasttree_oracle as oracle
    from fasttree_hip import launch_schedule
    from helpers import assert_parity

    rng = random.Random(7)
    hq, hkv, d = 32, 8, 128
    system = [rng.randint(1, 10**6) for _ in range(70)]
    prefixes, prompts, outputs = [system], [], []
    for _ in range(3):
        mid = system + [rng.randint(1, 10**6) for _ in range(33)]
        prefixes.append(mid)
        for _ in range(9):
            prompts.append(mid + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 20))])
            outputs.append([rng.randint(1, 10**6) for _ in range(rng.randint(0, 6))])
    n = len(prompts)
    rows = list(range(n))
    rng.shuffle(rows)
    batch, n_slots = make_batch(prompts, outputs, prefixes, device=device, max_ctx=256, row_of=rows)
    if joined == "reference_order":
        meta = small_meta(device=device, launch_order=False)
    elif joined in ("merged", "merged_reference_order"):
        # the cost model evaluated (fix_enumerate) with a reduction cost that merges every shared node
        meta = small_meta(device=device, fix_enumerate=True, gamma=50.0, para_threshs1=(0, 0), para_threshs2=(0, 0),
                          launch_order=joined == "merged")
    elif joined:
        monkeypatch.setattr(launch_schedule, "MIN_PROGRAM_TILES", 0.0)
        meta = small_meta(device=device, TSQs=(256 // 4, 16 // 4), kv_split_sizes=(32, 16))
    else:
        meta = small_meta(device=device, TSQs=(256 // 4, 16 // 4))
    prepare_for_fasttree_meta(batch, meta)
    print("\n[gpu case] hook", dtype, "joined" if joined else "as planned", "vnodes", list(meta.phase_node_nums), flush=True)

    g = torch.Generator().manual_seed(3)
    k_pool = torch.randn((n_slots + 8, hkv, d), generator=g).to(dtype).to(device)
    v_pool = torch.randn((n_slots + 8, hkv, d), generator=g).to(dtype).to(device)
    q = torch.randn((n, hq * d), generator=g).to(dtype).to(device)
    k_new = torch.randn((n, hkv * d), generator=g).to(dtype).to(device)
    v_new = torch.randn((n, hkv * d), generator=g).to(dtype).to(device)
    table = batch.req_to_token_pool.req_to_token
    lens = [len(p) + len(o) + 1 for p, o in zip(prompts, outputs)]
    out_loc = torch.tensor([int(table[rows[r], lens[r] - 1]) for r in range(n)], device=device)
    im = Obj(token_to_kv_pool=FakePool(k_pool, v_pool), req_to_token_pool=batch.req_to_token_pool,
             fasttree=meta, out_cache_loc=out_loc)
    layer = FakeLayer(hq, hkv, d)
    layer.decode_forward = decode_forward_fasttree.__get__(layer)
    o = layer.decode_forward(q, k_new, v_new, im)
    torch.cuda.synchronize()
    assert o.shape == q.shape and o.dtype == dtype
    paths = [table[rows[r], : lens[r]].cpu().long() for r in range(n)]
    want = oracle.dense_attention(q.view(n, hq, d).cpu(), k_pool.cpu(), v_pool.cpu(), paths, layer.scaling)
    assert_parity(o.view(n, hq, d).cpu(), want, "hook", out_dtype=dtype)

    # one more token per request: grow the last vnodes in place, as between two decode steps
    for r in range(n):
        table[rows[r], lens[r]] = n_slots + 0  # any valid slot; every request gets the same new row here
    k_pool[n_slots] = torch.randn((hkv, d), generator=g).to(dtype).to(device)
    v_pool[n_slots] = torch.randn((hkv, d), generator=g).to(dtype).to(device)
    prepare_for_fasttree_step(batch, meta)
    im.out_cache_loc = torch.full((n,), n_slots, device=device)
    o2 = layer.decode_forward(q, k_pool[n_slots].reshape(1, -1).expand(n, -1).contiguous(),
                              v_pool[n_slots].reshape(1, -1).expand(n, -1).contiguous(), im)
    torch.cuda.synchronize()
    paths2 = [table[rows[r], : lens[r] + 1].cpu().long() for r in range(n)]
    want2 = oracle.dense_attention(q.view(n, hq, d).cpu(), k_pool.cpu(), v_pool.cpu(), paths2, layer.scaling)
    assert_parity(o2.view(n, hq, d).cpu(), want2, "hook after step", out_dtype=dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("loc_dtype", [torch.int32, torch.int64])
def test_store_kv_cache_equals_the_two_indexed_assignments(device, dtype, loc_dtype):
    """One launch for both pools against torch's indexed assignment, bit for bit: flat and
    three-dimensional new rows, rows that are a slice of a wider tensor (qkv projections), pools
    with padded slot strides, int32 and int64 slots; slots outside the pool are skipped."""
    from fasttree_hip.decode import store_kv_cache

    g = torch.Generator().manual_seed(5)
    hkv, d, slots, n = 8, 128, 500, 37
    wide_k = torch.randn((slots, hkv + 2, d), generator=g).to(dtype).to(device)
    k_pool, v_pool = wide_k[:, 1:-1], torch.randn((slots, hkv, d), generator=g).to(dtype).to(device)
    qkv = torch.randn((n, 3 * hkv * d), generator=g).to(dtype).to(device)
    k_new, v_new = qkv[:, hkv * d: 2 * hkv * d], qkv[:, 2 * hkv * d:]
    loc = torch.randperm(slots, generator=g)[:n].to(loc_dtype).to(device)
    want_k, want_v, want_wide = k_pool.clone(), v_pool.clone(), wide_k.clone()
    want_k[loc.long()] = k_new.reshape(n, hkv, d)
    want_v[loc.long()] = v_new.reshape(n, hkv, d)
    store_kv_cache(k_new, v_new, loc, k_pool, v_pool)
    torch.cuda.synchronize()
    assert torch.equal(k_pool, want_k) and torch.equal(v_pool, want_v)
    assert torch.equal(wide_k[:, 0], want_wide[:, 0]) and torch.equal(wide_k[:, -1], want_wide[:, -1])
    # out of range: skipped, everything else written
    loc2 = loc.clone()
    loc2[3], loc2[11] = slots, -1
    k_new2 = torch.randn((n, hkv, d), generator=g).to(dtype).to(device)
    keep = torch.ones(n, dtype=torch.bool)
    keep[3] = keep[11] = False
    want_k[loc[keep.to(device)].long()] = k_new2[keep.to(device)]
    want_v[loc[keep.to(device)].long()] = k_new2[keep.to(device)]
    store_kv_cache(k_new2, k_new2.clone(), loc2, k_pool, v_pool)
    torch.cuda.synchronize()
    assert torch.equal(k_pool, want_k) and torch.equal(v_pool, want_v)
    store_kv_cache(k_new2[:0], k_new2[:0], loc2[:0], k_pool, v_pool)  # no tokens: nothing to do
    with pytest.raises(Exception):
        store_kv_cache(k_new2.float(), k_new2.float(), loc2, k_pool, v_pool)
    with pytest.raises(Exception):
        store_kv_cache(k_new2, k_new2, loc2[:5], k_pool, v_pool)


@pytest.mark.gpu
def test_hook_with_the_fused_store(device):
    """FastTreeMetadata(fused_store=True): the hook writes the new rows itself (the layer's
    store_kv_cache is not called) and attends them."""
    import fasttree_oracle as oracle
    from helpers import assert_parity

    rng = random.Random(9)
    hq, hkv, d, dtype = 32, 8, 128, torch.float16
    system = [rng.randint(1, 10**6) for _ in range(50)]
    prompts = [system + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 30))] for _ in range(12)]
    outputs = [[rng.randint(1, 10**6) for _ in range(rng.randint(0, 4))] for _ in prompts]
    n = len(prompts)
    batch, n_slots = make_batch(prompts, outputs, [system], device=device, max_ctx=128)
    meta = small_meta(device=device, fused_store=True)
    prepare_for_fasttree_meta(batch, meta)
    g = torch.Generator().manual_seed(4)
    k_pool = torch.randn((n_slots + 8, hkv, d), generator=g).to(dtype).to(device)
    v_pool = torch.randn((n_slots + 8, hkv, d), generator=g).to(dtype).to(device)
    q = torch.randn((n, hq * d), generator=g).to(dtype).to(device)
    k_new = torch.randn((n, hkv * d), generator=g).to(dtype).to(device)
    v_new = torch.randn((n, hkv * d), generator=g).to(dtype).to(device)
    table = batch.req_to_token_pool.req_to_token
    lens = [len(p) + len(o) + 1 for p, o in zip(prompts, outputs)]
    out_loc = torch.tensor([int(table[r, lens[r] - 1]) for r in range(n)], device=device, dtype=torch.int32)
    im = Obj(token_to_kv_pool=FakePool(k_pool, v_pool), req_to_token_pool=batch.req_to_token_pool,
             fasttree=meta, out_cache_loc=out_loc)
    layer = FakeLayer(hq, hkv, d)

    def refuse(*a, **k):
        raise AssertionError("the layer's store_kv_cache must not be called")
    layer.store_kv_cache = refuse
    layer.decode_forward = decode_forward_fasttree.__get__(layer)
    o = layer.decode_forward(q, k_new, v_new, im)
    torch.cuda.synchronize()
    assert torch.equal(k_pool[out_loc.long()], k_new.view(n, hkv, d)) and torch.equal(v_pool[out_loc.long()], v_new.view(n, hkv, d))
    paths = [table[r, : lens[r]].cpu().long() for r in range(n)]
    want = oracle.dense_attention(q.view(n, hq, d).cpu(), k_pool.cpu(), v_pool.cpu(), paths, layer.scaling)
    assert_parity(o.view(n, hq, d).cpu(), want, "hook, fused store", out_dtype=dtype)


def test_plan_is_reused_only_for_the_very_same_requests():
    """The hook re-plans unless the batch holds, one by one, the request objects the plan was
    made for; the kept tuple owns them, so an address cannot come back under a new request."""
    from fasttree_hip.sglang_plugin import same_requests
    a, b, c = Obj(), Obj(), Obj()
    kept = (a, b)
    assert same_requests(kept, [a, b]) and same_requests(kept, (a, b))
    assert not same_requests(None, [a, b]) and not same_requests(kept, [b, a])
    assert not same_requests(kept, [a]) and not same_requests(kept, [a, b, c]) and not same_requests(kept, [a, c])
    twin = Obj()
    twin.__dict__.update(b.__dict__)
    assert not same_requests(kept, [a, twin]), "equal contents are not the same request"
    assert same_requests((), [])


@pytest.mark.parametrize("launch_order", [False, True])
@pytest.mark.parametrize("gamma", [0.1, 50.0])
@pytest.mark.parametrize("seed", range(6))
def test_merge_path_keeps_what_every_request_attends(seed, gamma, launch_order):
    """FastTreeMetadata(fix_enumerate=True): the cost model is evaluated and nodes are merged
    into their children (with a large gamma: wherever the model is asked).  Whatever it decides,
    every request attends each of its tokens exactly once through the rows listed for it --
    also requests whose prompt ends at an inner node of the radix tree -- and its last vnode is
    still the single-request vnode that ends where its tokens end."""
    rng = random.Random(500 + seed)
    system = [rng.randint(1, 10**6) for _ in range(rng.randint(5, 90))]
    prefixes, prompts, outputs = [system], [], []
    for _ in range(rng.randint(1, 4)):
        mid = system + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 60))]
        prefixes.append(mid)
        if rng.random() < 0.5:
            prompts.append(list(mid)); outputs.append([rng.randint(1, 10**6) for _ in range(rng.randint(0, 9))])   # ends at an inner node
        for _ in range(rng.randint(1, 12)):
            prompts.append(mid + [rng.randint(1, 10**6) for _ in range(rng.randint(1, 40))])
            outputs.append([rng.randint(1, 10**6) for _ in range(rng.randint(0, 12))])
    batch, _ = make_batch(prompts, outputs, prefixes, max_ctx=256)
    meta = small_meta(kv_split_sizes=(16, 8), gamma=gamma, fix_enumerate=True, launch_order=launch_order)
    prepare_for_fasttree_meta(batch, meta)
    table = batch.req_to_token_pool.req_to_token
    got = plan_lists(meta, batch)
    for r, slots in enumerate(covered_slots(meta, batch)):
        assert sorted(slots) == sorted(table[r, : len(prompts[r]) + len(outputs[r]) + 1].tolist()), r
        rows = got["req_entries"][got["req_offs"][r]: got["req_offs"][r] + got["req_lens"][r]]
        assert rows == sorted(set(rows)) and all(got["q_entries"][i] == r for i in rows)
        v = meta.req_last_vnodes[r]
        assert got["q_lens"][v] == 1 and got["q_entries"][got["q_offs"][v]] == r
        assert got["kv_offs"][v] + got["kv_lens"][v] == r * table.stride(0) + len(prompts[r]) + len(outputs[r]) + 1
    assert sum(got["req_lens"]) == len(got["q_entries"])


def test_merge_path_hand_derived():
    """A=[1,2,3,4] -> B=[5,6] (request 0), C=[7,8,9] (requests 1, 2).  With a reduction cost of
    50 per query the model merges A into both children: request 0 attends A+B as one run of 6
    tokens through its own row, requests 1 and 2 attend A+C as one run of 7 through the row of
    request 1; A keeps no vnode.  With the default cost (0.1) nothing is merged and the plan is
    the shipped one."""
    prompts = [[1, 2, 3, 4, 5, 6], [1, 2, 3, 4, 7, 8, 9], [1, 2, 3, 4, 7, 8, 9]]
    outputs = [[10, 11], [12], []]
    batch, _ = make_batch(prompts, outputs, shared_prefixes=[[1, 2, 3, 4]], row_of=[2, 0, 5])
    s = 64
    # (thresholds of 0: the tile sizes stay as given; with the default thresholds this small batch
    # ends up with 16-request tiles, for which the model does not merge)
    meta = small_meta(launch_order=False, fix_enumerate=True, gamma=50.0, para_threshs1=(0, 0), para_threshs2=(0, 0))
    prepare_for_fasttree_meta(batch, meta)
    got = plan_lists(meta, batch)
    assert got["kv_offs"] == [2 * s + 0, 0 * s + 0, 2 * s + 6, 0 * s + 7, 5 * s + 7]
    assert got["kv_lens"] == [6, 7, 3, 2, 1]
    assert got["q_lens"] == [1, 2, 1, 1, 1] and got["q_entries"] == [0, 1, 2, 0, 1, 2]
    assert got["req_lens"] == [2, 2, 2] and meta.req_last_vnodes == [2, 3, 4]
    shipped, same = small_meta(launch_order=False), small_meta(launch_order=False, fix_enumerate=True)
    prepare_for_fasttree_meta(batch, shipped)
    prepare_for_fasttree_meta(batch, same)
    assert plan_lists(same, batch) == plan_lists(shipped, batch)


def test_hook_replans_for_new_requests_and_every_few_forwards():
    """The decision the patched forward_decode_batch takes, with stand-ins for the server and the
    requests: a new plan for a batch of other request objects -- also when a finished request was
    freed and a new one may sit at its address --, the +1 step while the batch is unchanged, and
    a new plan after `replan_every` forwards (the reference plans once per forward_step and steps
    between its num_continue_decode_steps forwards, plugin.py:108-131)."""
    import gc
    from fasttree_hip.sglang_plugin import plan_or_step
    calls = []
    plan = lambda batch, meta: calls.append("plan")
    step = lambda batch, meta: calls.append("step")
    server = Obj(fasttree_metadata=object(), _fasttree_planned_for=None, _fasttree_forwards=0)
    a, b = Req([1], []), Req([2], [])
    batch = Obj(reqs=[a, b])
    assert [plan_or_step(server, batch, 3, plan, step) for _ in range(7)] == ["plan", "step", "step", "plan", "step", "step", "plan"]
    batch.reqs = [a]                              # a request finished
    assert plan_or_step(server, batch, 3, plan, step) == "plan"
    # batch size 1 served back to back: the old request is freed before the new one is made
    del a, b
    batch.reqs = [Req([3], [])]
    seen = set()
    for _ in range(50):
        assert plan_or_step(server, batch, 100, plan, step) == "plan"
        seen.add(id(batch.reqs[0]))
        batch.reqs = []                           # the only other holder lets go ...
        gc.collect()
        batch.reqs = [Req([4], [])]               # ... and a new request is made, possibly at the same address
    assert calls.count("plan") == 54 and calls.count("step") == 4


# ---- the loader, with stand-ins for the SGLang modules it patches
def _install_sglang_stubs(monkeypatch, continue_steps=3):
    """Modules with the names and the few members load_fasttree_plugin touches (SGLang v0.2.13:
    RadixAttention, ModelTpServer, InputMetadata.from_schedule_batch, global_config); each records
    what the patched versions hand on to it."""
    import sys
    import types

    log = []

    class RadixAttention:
        def __init__(self, num_heads, head_dim, scaling, num_kv_heads, layer_id):
            self.tp_q_head_num, self.qk_head_dim, self.v_head_dim = num_heads, head_dim, head_dim
            self.scaling, self.layer_id, self.logit_cap = scaling, layer_id, -1

        def decode_forward(self, q, k, v, input_metadata):
            return "sglang decode"

    class ModelTpServer:
        def __init__(self, gpu_id, tp_rank, server_args, nccl_port, model_overide_args):
            log.append(("server init", server_args.disable_cuda_graph))
            self.gpu_id, self.tp_rank = gpu_id, tp_rank
            self.model_config = Obj(num_attention_heads=32, num_key_value_heads=8, head_dim=128)

        def forward_prefill_batch(self, batch):
            log.append(("prefill", batch))
            return "prefilled"

        def forward_decode_batch(self, batch):
            log.append(("decode", batch))
            return "decoded"

    class InputMetadata:
        @classmethod
        def from_schedule_batch(cls, model_runner, batch, forward_mode):
            ret = cls()
            ret.made_from = (model_runner, batch, forward_mode)
            return ret

    def module(name, **members):
        mod = types.ModuleType(name)
        mod.__dict__.update(members)
        monkeypatch.setitem(sys.modules, name, mod)
        return mod

    module("sglang")
    module("sglang.srt")
    module("sglang.srt.layers")
    module("sglang.srt.layers.radix_attention", RadixAttention=RadixAttention)
    module("sglang.srt.managers")
    module("sglang.srt.managers.tp_worker", ModelTpServer=ModelTpServer)
    module("sglang.srt.model_executor")
    module("sglang.srt.model_executor.forward_batch_info", InputMetadata=InputMetadata)
    module("sglang.global_config", global_config=Obj(num_continue_decode_steps=continue_steps))
    # (the reference's own plugin package must not be found: its loader would be used instead)
    monkeypatch.setitem(sys.modules, "fasttree_sglang_plugin_v0_2_13", None)
    return Obj(RadixAttention=RadixAttention, ModelTpServer=ModelTpServer, InputMetadata=InputMetadata, log=log)


@pytest.mark.parametrize("annotate", [False, True])
def test_loader_patches_the_three_sglang_classes(monkeypatch, annotate):
    """load_fasttree_plugin without the reference's plugin package (plugin.py:190-238): every
    RadixAttention instance gets the hook bound as its decode_forward, InputMetadata carries the
    batch's metadata as .fasttree, ModelTpServer switches graphs off, creates the metadata from
    its model config and, before every decode forward, plans (new requests, or the plan has served
    num_continue_decode_steps forwards) or steps."""
    import fasttree_hip.sglang_plugin as plugin

    sg = _install_sglang_stubs(monkeypatch, continue_steps=3)
    made = []

    class Metadata:
        def __init__(self, num_qo_heads, num_kv_heads, head_dim, device):
            made.append((num_qo_heads, num_kv_heads, head_dim, str(device)))

    planned = []
    monkeypatch.setattr(plugin, "FastTreeMetadata", Metadata)
    monkeypatch.setattr(plugin, "prepare_for_fasttree_meta", lambda batch, meta: planned.append(("plan", batch, meta)))
    monkeypatch.setattr(plugin, "prepare_for_fasttree_step", lambda batch, meta: planned.append(("step", batch, meta)))
    # the patched classes are this test's own stand-ins: nothing to restore but the module's two functions
    plugin.load_fasttree_plugin(True, annotate)

    layer = sg.RadixAttention(32, 128, 0.088, 8, layer_id=5)
    assert layer.decode_forward.__func__ is plugin.decode_forward_fasttree and layer.decode_forward.__self__ is layer
    other = sg.RadixAttention(32, 128, 0.088, 8, layer_id=6)
    assert other.decode_forward.__self__ is other          # bound per instance, as plugin.py:58 does

    meta = object()
    batch = Obj(reqs=[Req([1], []), Req([2], [])], fasttree_metadata=meta)
    im = sg.InputMetadata.from_schedule_batch("runner", batch, "DECODE")
    assert im.fasttree is meta and im.made_from == ("runner", batch, "DECODE")
    assert sg.InputMetadata.from_schedule_batch("runner", Obj(reqs=[]), "EXTEND").fasttree is None

    args = Obj(disable_cuda_graph=False)
    server = sg.ModelTpServer(1, 0, args, 28000, {})
    assert args.disable_cuda_graph is True and sg.log[0] == ("server init", True)   # set before SGLang's own init runs
    assert made == [(32, 8, 128, "cuda:1")]
    assert isinstance(server.fasttree_metadata, Metadata)

    assert [server.forward_decode_batch(batch) for _ in range(4)] == ["decoded"] * 4
    assert [p[0] for p in planned] == ["plan", "step", "step", "plan"]
    assert all(p[1] is batch and p[2] is server.fasttree_metadata for p in planned)
    batch.reqs = batch.reqs[:1]                      # a request finished: other requests, a new plan
    server.forward_decode_batch(batch)
    assert planned[-1][0] == "plan"
    assert [e[0] for e in sg.log].count("decode") == 5  # SGLang's own forward still runs, after the plan
    assert server.forward_prefill_batch(batch) == "prefilled"
    if annotate:
        assert hasattr(sg.ModelTpServer.forward_prefill_batch, "__wrapped__")


def test_loader_does_nothing_when_everything_is_off(monkeypatch, capsys):
    import fasttree_hip.sglang_plugin as plugin

    sg = _install_sglang_stubs(monkeypatch)
    before = (sg.RadixAttention.__init__, sg.ModelTpServer.__init__, sg.ModelTpServer.forward_decode_batch)
    plugin.load_fasttree_plugin(False, False)
    assert "[Warning] FastTree plugin is not enabled" in capsys.readouterr().out        # plugin.py:235-237
    assert before == (sg.RadixAttention.__init__, sg.ModelTpServer.__init__, sg.ModelTpServer.forward_decode_batch)
    # the breakdown alone wraps SGLang's two forwards and leaves the attention path as it is
    plugin.load_fasttree_plugin(False, True)
    assert hasattr(sg.ModelTpServer.forward_decode_batch, "__wrapped__")
    assert sg.RadixAttention(32, 128, 0.088, 8, 0).decode_forward(None, None, None, None) == "sglang decode"


def test_loader_needs_sglang(monkeypatch):
    import sys
    import fasttree_hip.sglang_plugin as plugin
    for name in ("fasttree_sglang_plugin_v0_2_13", "sglang", "sglang.srt.layers.radix_attention"):
        monkeypatch.setitem(sys.modules, name, None)
    with pytest.raises(ImportError):
        plugin.load_fasttree_plugin(True, False)
