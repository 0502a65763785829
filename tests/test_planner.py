"""Host planner, tree utilities and input builder (CPU only)."""

import os

import numpy as np
import pytest

from cases import PLANNER_CASES, build_tree, digest
from fasttree_hip import kv_tree
from fasttree_hip.planner import FastTreeParams, _Cmm, _CpadK, _CpadQ, _tree_heuristic, fasttree_plan
from helpers import params_for, planner_goldens, run_planner

ARRAYS = ["vnode_to_kv_entries", "vnode_to_kv_offs", "vnode_to_kv_lens", "vnode_to_q_entries", "vnode_to_q_offs",
          "vnode_to_q_lens", "req_to_vnode_entries", "req_to_vnode_offs", "req_to_vnode_lens", "node_assignments"]


@pytest.fixture(scope="module")
def goldens():
    return planner_goldens()


@pytest.mark.parametrize("backend", ["python", "native"])
@pytest.mark.parametrize("case", PLANNER_CASES, ids=[c["name"] for c in PLANNER_CASES])
def test_planner_matches_reference_fixture(case, backend, goldens):
    """Every list, the mutated tile sizes and the printed lines equal what the reference
    planner produced for the same arguments -- for the Python planner and for the C++ one."""
    gold = goldens[case["name"]]
    _, _, batch, plan, params, text = run_planner(case, backend=backend)
    assert batch == gold["batch_size"]
    for name in ARRAYS:
        arr = np.asarray(getattr(plan, name), dtype=np.int32)
        assert arr.size == gold[name]["len"], name
        if "values" in gold[name]:
            assert arr.tolist() == gold[name]["values"], name
        else:
            assert arr[:64].tolist() == gold[name]["head"] and arr[-64:].tolist() == gold[name]["tail"], name
        assert digest(arr) == gold[name]["sha256"], name
    assert plan.phase_node_nums == gold["phase_node_nums"]
    assert plan.phase_node_offsets == gold["phase_node_offsets"]
    assert list(params.TSQs) == gold["final_TSQs"] and list(params.TSKs) == gold["final_TSKs"]
    assert text == gold["stdout"]
    assert [len(plan.vnode_to_q_entries), case["Hq"], case["D"]] == gold["mid_o_shape"]


def test_cost_function_known_answers():
    assert _CpadQ(16, 0) == 0 and _CpadQ(16, 16) == 0 and _CpadQ(16, 17) == 15 and _CpadQ(4, 1) == 3
    assert _CpadK(32, 40) == 0 and _CpadK(32, 8) == 24
    p = FastTreeParams()
    p.set_q_tile_sizes([64, 16]); p.set_kv_tile_sizes([32, 32])
    assert _Cmm(0, 123, p) == 0
    # one query, 100 keys, phase 1: alpha * 15 * 1 * 100
    assert _Cmm(1, 100, p) == pytest.approx(0.66 * 15 * 100)


def test_hand_derived_plan_kat1():
    """Three-level chain 100 -> 50 -> (10, 10): the middle node absorbs the root."""
    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": [1, 1, 2], "lens": [100, 50, 10]})
    p = FastTreeParams()
    p.set_values(0.66, 0.33, 0.1); p.set_q_tile_sizes([64, 16]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(1)
    plan = fasttree_plan(tree, ptrs, batch, 32, [1024, 128], [132, 528], [132, 132], p)
    assert plan.node_assignments == [0, 1, 0, 0]
    assert plan.parallelisms == [[0, 96], [0, 128], [0, 128]]
    assert list(zip(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens)) == [
        (0, 128, 0, 2), (128, 22, 2, 2), (150, 10, 4, 1), (160, 10, 5, 1)]
    assert plan.vnode_to_kv_entries.tolist() == list(range(170)) + [-1] * 32
    assert plan.vnode_to_q_entries == [0, 1, 0, 1, 0, 1]
    assert plan.req_to_vnode_entries == [0, 2, 4, 1, 3, 5] + [-1] * 32
    assert plan.req_to_vnode_offs == [0, 3] and plan.req_to_vnode_lens == [3, 3]
    assert plan.phase_node_nums == [0, 4] and plan.phase_node_offsets == [0, 0]
    assert p.TSQs == [64, 64] and p.TSKs == [32, 32]


def test_hand_derived_plan_c1_and_c3():
    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": [1, 16], "lens": [1024, 128]})
    p = FastTreeParams()
    p.set_q_tile_sizes([64, 16]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(1)
    plan = fasttree_plan(tree, ptrs, batch, 32, [1024, 128], [132, 528], [132, 132], p)
    assert sum(plan.node_assignments) == 0 and plan.parallelisms == [[0, 544]]
    assert (plan.vnode_to_kv_offs[0], plan.vnode_to_kv_lens[0], plan.vnode_to_q_lens[0]) == (0, 1024, 16)
    for k in range(16):
        assert (plan.vnode_to_kv_offs[1 + k], plan.vnode_to_kv_lens[1 + k], plan.vnode_to_q_offs[1 + k]) == (
            1024 + 128 * k, 128, 16 + k)
        assert plan.req_to_vnode_entries[2 * k: 2 * k + 2] == [k, 16 + k]

    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": [1, 10, 400], "lens": [4000, 400, 40]})
    p = FastTreeParams()
    p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(4)
    plan = fasttree_plan(tree, ptrs, batch, 8, [1024, 128], [132, 528], [132, 132], p)
    assert sum(plan.node_assignments) == 0 and plan.parallelisms == [[1040, 3200]]
    assert plan.num_vnodes == 530 and plan.num_rows == 2400 and plan.phase_node_nums == [130, 400]


def _coverage(plan, tree, ptrs, batch):
    """For each request: the multiset of logical tokens its scratch rows attend."""
    row_vnodes = {}
    for v in range(plan.num_vnodes):
        for i in range(plan.vnode_to_q_lens[v]):
            row_vnodes.setdefault(plan.vnode_to_q_offs[v] + i, []).append(v)
    seen = [[] for _ in range(batch)]
    for row, req in enumerate(plan.vnode_to_q_entries):
        assert len(row_vnodes[row]) == 1, "a scratch row belongs to exactly one vnode"
        v = row_vnodes[row][0]
        off, ln = plan.vnode_to_kv_offs[v], plan.vnode_to_kv_lens[v]
        seen[req].extend(plan.vnode_to_kv_entries[off: off + ln].tolist())
    return seen


@pytest.mark.parametrize("name", ["kat1", "c1", "c3", "c5_seed0", "c5_seed1", "shape07_h32_8", "shape07_h16_1_gamma10",
                                  "rand03", "rand17", "rand41"])
def test_plan_invariants(name):
    """Each request attends every token of its root path exactly once, whatever the split."""
    case = next(c for c in PLANNER_CASES if c["name"] == name)
    tree, ptrs, batch, plan, params, _ = run_planner(case)
    seen = _coverage(plan, tree, ptrs, batch)
    leaves = [i for i, t in enumerate(tree) if t.num_children == 0]
    for req, leaf in enumerate(leaves):
        want = []
        for node in kv_tree.root_path(tree, leaf):
            want.extend(range(ptrs[node], ptrs[node + 1]))
        assert sorted(seen[req]) == want
    assert sum(plan.vnode_to_q_lens) == plan.num_rows
    assert max(plan.vnode_to_q_lens) <= plan.q_tile_sizes[0]
    wide = plan.phase_node_nums[0]
    assert all(n > plan.q_tile_sizes[1] for n in plan.vnode_to_q_lens[:wide])
    assert all(n <= plan.q_tile_sizes[1] for n in plan.vnode_to_q_lens[wide:])
    total = len(plan.vnode_to_kv_entries) - 32
    assert all(o + n <= total for o, n in zip(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens))
    for r in range(batch):
        rows = plan.req_to_vnode_entries[plan.req_to_vnode_offs[r]: plan.req_to_vnode_offs[r] + plan.req_to_vnode_lens[r]]
        assert rows == sorted(rows) and all(plan.vnode_to_q_entries[x] == r for x in rows)


@pytest.mark.parametrize("case", PLANNER_CASES, ids=[c["name"] for c in PLANNER_CASES])
def test_preparation_returns_the_reference_lists_by_default(case, goldens):
    """The function that carries the reference's name, called as the reference is (no
    launch-order argument; `device` only because there is no GPU here), returns the reference's
    tuple: the nine index arrays, scratch of the reference's shapes, the two phase lists as plain
    lists, the assignments; it mutates `params` and prints as the reference does
    (kernel_bench/fasttree.py:99-296)."""
    import contextlib, io
    import torch
    from fasttree_hip.planner import fasttree_preparation
    gold = goldens[case["name"]]
    tree, ptrs, batch = build_tree(case["tree"])
    params = params_for(case)
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        aux, assignments = fasttree_preparation(tree, ptrs, batch, case["Hq"], case["Hkv"], case["D"],
                                                list(case["kv_split_sizes"]), list(case["para_threshs1"]),
                                                list(case["para_threshs2"]), params, device="cpu")
    assert len(aux) == 13
    for name, tensor in zip(ARRAYS[:9], aux[:9]):
        assert tensor.dtype == torch.int32 and tensor.numel() == gold[name]["len"], name
        assert digest(tensor.numpy()) == gold[name]["sha256"], name
    assert digest(np.asarray(assignments, dtype=np.int32)) == gold["node_assignments"]["sha256"]
    assert list(aux[9].shape) == gold["mid_o_shape"] and aux[9].dtype == torch.float32
    assert list(aux[10].shape) == gold["mid_o_shape"][:2] and aux[10].dtype == torch.float32
    assert type(aux[11]) is list and aux[11] == gold["phase_node_nums"]
    assert type(aux[12]) is list and aux[12] == gold["phase_node_offsets"]
    assert list(params.TSQs) == gold["final_TSQs"] and list(params.TSKs) == gold["final_TSKs"]
    assert out.getvalue() == gold["stdout"]


def test_preparation_into_preallocated_buffers():
    """fasttree_preparation(buffers=...) writes into the same device buffers on every call and
    returns their leading parts; the contents equal those of the allocating call."""
    import torch
    from fasttree_hip.planner import FastTreeParams, PlanBuffers, fasttree_preparation
    buffers = PlanBuffers(32, 128, max_kv_entries=400000, max_rows=8192, max_vnodes=8192, max_batch_size=2048, device="cpu")
    ptrs_seen = None
    for name in ("c3", "c1", "shape07_h32_8"):
        case = next(c for c in PLANNER_CASES if c["name"] == name)
        tree, ptrs, batch = build_tree(case["tree"])
        outs = []
        for buf in (None, buffers):
            params = FastTreeParams()
            params.set_values(case["alpha"], case["beta"], case["gamma"]); params.set_q_tile_sizes(list(case["TSQs"]))
            params.set_kv_tile_sizes(list(case["TSKs"])); params.set_kv_group_num(case["Hq"] // case["Hkv"])
            if case["Hq"] != 32:
                continue
            outs.append(fasttree_preparation(tree, ptrs, batch, case["Hq"], case["Hkv"], 128, list(case["kv_split_sizes"]),
                                             list(case["para_threshs1"]), list(case["para_threshs2"]), params,
                                             device="cpu", buffers=buf))
        if len(outs) < 2:
            continue
        (a, assign_a), (b, assign_b) = outs
        assert assign_a == assign_b and a[11] == b[11] and a[12] == b[12]
        for i in range(9):
            assert torch.equal(a[i], b[i]), i
        assert b[9].shape == a[9].shape and b[10].shape == a[10].shape
        now = [t.data_ptr() for t in b[:11]]
        assert ptrs_seen is None or now == ptrs_seen, "every call writes into the same buffers"
        ptrs_seen = now
    assert ptrs_seen is not None
    small = PlanBuffers(32, 128, max_kv_entries=100, max_rows=4096, max_vnodes=2048, max_batch_size=512, device="cpu")
    case = next(c for c in PLANNER_CASES if c["name"] == "c3")
    tree, ptrs, batch = build_tree(case["tree"])
    params = FastTreeParams()
    params.set_values(0.66, 0.33, 0.1); params.set_q_tile_sizes([16, 4]); params.set_kv_tile_sizes([32, 32]); params.set_kv_group_num(4)
    with pytest.raises(ValueError):
        fasttree_preparation(tree, ptrs, batch, 32, 8, 128, [1024, 128], [132, 528], [132, 132], params, device="cpu", buffers=small)


def test_ablation_extremes():
    """gamma = +10 with alpha = beta = 0 merges every node into its leaf path (one vnode per
    request over its whole path); gamma = -10 never merges."""
    spec = {"kind": "regular", "sizes": [1, 4, 16], "lens": [100, 30, 7]}
    for gamma, expect in ((10.0, 1), (-10.0, 0)):
        tree, ptrs, batch = build_tree(spec)
        p = FastTreeParams()
        p.set_values(0.0, 0.0, gamma); p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(4)
        assign = _tree_heuristic(tree, p)
        assert assign[0] == 0 and all(a == expect for a in assign[1:])


def test_single_child_chain_always_merges():
    rows = [[-1, 0, 50, 1], [0, 1, 20, 1], [1, 2, 9, 1], [2, 3, 4, 0]]
    tree = kv_tree.nodes_from_rows(rows)
    kv_tree.assign_requests(tree)
    p = FastTreeParams()
    p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(4)
    assert _tree_heuristic(tree, p) == [0, 1, 1, 1]


def test_native_planner_rejects_bad_trees():
    from fasttree_hip import _plan_lib
    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": [1, 2], "lens": [8, 8]})
    p = FastTreeParams()
    p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32])
    args = (batch, 8, [1024, 128], [132, 528], [132, 132], 0.66, 0.33, 0.1)
    with pytest.raises(_plan_lib.FastTreePlannerError):
        _plan_lib.plan(tree, ptrs[:-1], *args, p.TSQs, p.TSKs, 1)               # wrong prefix-sum length
    with pytest.raises(_plan_lib.FastTreePlannerError):
        _plan_lib.plan(tree, ptrs, *args, [0, 4], p.TSKs, 1)                    # tile size 0
    tree[1].requests = [batch + 3]
    with pytest.raises(_plan_lib.FastTreePlannerError):
        _plan_lib.plan(tree, ptrs, *args, p.TSQs, p.TSKs, 1)                    # request id out of range


@pytest.mark.parametrize("backend", ["python", "native"])
def test_backends_agree_on_slot_maps_and_big_trees(backend):
    case = next(c for c in PLANNER_CASES if c["name"] == "c4")
    _, ptrs, _, plain, _, _ = run_planner(case, backend=backend)
    perm = np.random.default_rng(5).permutation(ptrs[-1]).astype(np.int32)
    _, _, _, mapped, _, _ = run_planner(case, kv_slot_map=perm, backend=backend)
    assert np.array_equal(mapped.vnode_to_kv_entries[:-32], perm[plain.vnode_to_kv_entries[:-32]])
    assert digest(np.asarray(mapped.vnode_to_kv_entries, dtype=np.int32)) == {
        "python": digest, "native": digest}[backend](np.concatenate([perm[plain.vnode_to_kv_entries[:-32]],
                                                                     np.full(32, -1, np.int32)]).astype(np.int32))


def test_slot_map_is_an_indirection():
    case = next(c for c in PLANNER_CASES if c["name"] == "c5_seed2")
    _, ptrs, _, plain, _, _ = run_planner(case)
    perm = np.random.default_rng(3).permutation(ptrs[-1])
    _, _, _, mapped, _, _ = run_planner(case, kv_slot_map=perm)
    assert (mapped.vnode_to_kv_entries[:-32] == perm[plain.vnode_to_kv_entries[:-32]]).all()
    assert mapped.vnode_to_kv_entries[-32:].tolist() == [-1] * 32
    assert mapped.vnode_to_kv_offs == plain.vnode_to_kv_offs


def test_regular_generator_closed_form(tmp_path):
    rows = kv_tree.generate_tree([1, 3, 7], [5, 4, 3])
    assert [r[0] for r in rows] == [-1, 0, 0, 0] + [1 + (j * 3) // 7 for j in range(7)]
    assert [r[1] for r in rows] == list(range(11))
    assert [r[2] for r in rows] == [5] + [4] * 3 + [3] * 7
    assert [r[3] for r in rows] == [3, 3, 2, 2] + [0] * 7
    with pytest.raises(ValueError):
        kv_tree.generate_tree([1, 2], [3])
    path = os.path.join(tmp_path, "t.txt")
    kv_tree.save_tree(rows, path)
    assert open(path).read().splitlines()[:3] == ["11", "-1 0 5 3", "0 1 4 3"]
    back = kv_tree.retrive_from_file(path)
    assert [[t.parent, t.id, t.seqlen, t.num_children] for t in back] == rows
    assert all(t.requests == [] for t in back)


def test_request_numbering_and_prefix_sums():
    tree = kv_tree.nodes_from_rows(kv_tree.generate_tree([1, 2, 4], [10, 5, 2]))
    assert kv_tree.assign_requests(tree) == 4
    assert tree[0].requests == [0, 1, 2, 3] and tree[1].requests == [0, 1] and tree[2].requests == [2, 3]
    assert [tree[i].requests for i in range(3, 7)] == [[0], [1], [2], [3]]
    assert kv_tree.kv_prefix_sums(tree) == [0, 10, 15, 20, 22, 24, 26, 28]


def test_irregular_generator_properties():
    for seed in range(4):
        rows = kv_tree.generate_irregular_tree(seed)
        assert rows == kv_tree.generate_irregular_tree(seed)
        leaves = sum(1 for r in rows if r[3] == 0)
        assert 1 <= leaves <= 1024
        assert all(16 <= r[2] <= 2048 for r in rows)
        assert all(r[0] < r[1] for r in rows) and rows[0][0] == -1
        counts = [0] * len(rows)
        for r in rows[1:]:
            counts[r[0]] += 1
        assert counts == [r[3] for r in rows] and max(counts) <= 8
        depth = [0] * len(rows)
        for r in rows[1:]:
            depth[r[1]] = depth[r[0]] + 1
        assert max(depth) <= 4


def test_input_builder_paths_and_gather():
    import torch
    from fasttree_hip.inputs import gather_per_request, make_decode_inputs, qkv_preparation

    tree = kv_tree.nodes_from_rows(kv_tree.generate_tree([1, 2, 4], [6, 3, 2]))
    inp = make_decode_inputs(tree, 4, 2, 32, device="cpu", dtype=torch.float16, seed=5, shuffle_slots=True)
    again = make_decode_inputs(tree, 4, 2, 32, device="cpu", dtype=torch.float16, seed=5, shuffle_slots=True)
    assert torch.equal(inp.K_pool, again.K_pool) and torch.equal(inp.Q, again.Q)
    assert sorted(inp.slot_map.tolist()) == list(range(20))
    plain = make_decode_inputs(tree, 4, 2, 32, device="cpu", dtype=torch.float16, seed=5, shuffle_slots=False)
    assert torch.equal(inp.K_pool[torch.from_numpy(inp.slot_map)], plain.K_pool)
    k_cache, v_cache, lens = gather_per_request(inp)
    assert lens.tolist() == [11, 11, 11, 11] and k_cache.shape == (4, 11, 2, 32)
    assert torch.equal(k_cache[2, :6], plain.K_pool[0:6]) and torch.equal(k_cache[2, 6:9], plain.K_pool[9:12])
    assert torch.equal(v_cache[3, 9:11], plain.V_pool[18:20])
    out = qkv_preparation(tree, 4, 2, 32, "cpu", torch.float16, seed=5)
    assert len(out) == 7 and out[6] == [0, 6, 9, 12, 14, 16, 18, 20] and torch.equal(out[4], plain.K_pool)
