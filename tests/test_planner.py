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


@pytest.mark.parametrize("light_work", [0, 4096, 1 << 40])
@pytest.mark.parametrize("name", ["kat1", "c3", "c5_seed0", "rand17", "shape07_h32_8"])
def test_launch_order_is_a_permutation_of_the_vnodes(name, light_work):
    """The launch order keeps the vnode tuples; first-phase vnodes of at most light_work rows x
    tokens join the second phase, which is listed by decreasing tokens x passes with ties in the
    previous order; the other first-phase vnodes keep their order."""
    from fasttree_hip.planner import vnodes_in_launch_order
    case = next(c for c in PLANNER_CASES if c["name"] == name)
    tree, ptrs, batch, plan, params, _ = run_planner(case)
    group = case["Hq"] // case["Hkv"]
    before = list(zip(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens))
    *lists, nums, offs = vnodes_in_launch_order(
        plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
        plan.phase_node_nums, plan.phase_node_offsets, group, light_work=light_work)
    after = list(zip(*(x.tolist() for x in lists)))
    wide = plan.phase_node_nums[0]
    light = lambda v: v[1] * v[3] * group <= light_work and v[3] * group <= 64
    work = lambda v: v[1] * ((v[3] * group + 15) // 16)
    stay = [v for v in before[:wide] if not light(v)]
    move = [v for v in before[:wide] if light(v)]
    assert nums == [len(stay), len(before) - len(stay)] and offs == [0, len(stay)]
    assert after[:nums[0]] == stay
    assert after[nums[0]:] == sorted(move + before[wide:], key=lambda v: -work(v))  # (sorted() is stable)
    assert sorted(after) == sorted(before)
    assert list(plan.vnode_to_kv_lens) == [v[1] for v in before], "the plan itself is not touched"
    if light_work == 0:
        assert nums == list(plan.phase_node_nums)
    # with the number of kv heads given, nothing moves unless the first phase oversubscribes the machine
    *_, nums_few, _ = vnodes_in_launch_order(
        plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
        plan.phase_node_nums, plan.phase_node_offsets, group, 1, light_work=light_work)
    assert nums_few == (nums if wide > 512 else list(plan.phase_node_nums))


@pytest.mark.parametrize("name", ["c3", "c5_seed0", "shape07_h32_8", "rand17", "rand41"])
def test_launch_order_joins_query_tiles_without_changing_what_is_computed(name):
    """With the query tile given, neighbouring tiles of one run become one vnode of at most 128
    rows x chunks: every (run, scratch row) pair is still served exactly once."""
    from fasttree_hip.planner import vnodes_in_launch_order
    case = next(c for c in PLANNER_CASES if c["name"] == name)
    tree, ptrs, batch, plan, params, _ = run_planner(case)
    group = case["Hq"] // case["Hkv"]

    def pairs(kv_offs, kv_lens, q_offs, q_lens):
        out = []
        for ko, kl, qo, ql in zip(kv_offs, kv_lens, q_offs, q_lens):
            out.extend((int(ko), int(kl), int(qo) + i) for i in range(int(ql)))
        return sorted(out)

    before = pairs(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens)
    q_tile = plan.q_tile_sizes[0]
    *lists, nums, offs = vnodes_in_launch_order(
        plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
        plan.phase_node_nums, plan.phase_node_offsets, group, None, light_work=0, q_tile=q_tile)
    assert pairs(*lists) == before
    assert len(set(p[2] for p in before)) == plan.num_rows == len(before)
    chunks = max(1, min(8, -(-q_tile * group // 128)))
    cap = 128 * chunks // group
    wide_q = lists[3][:nums[0]]
    assert nums[1] == plan.phase_node_nums[1] and nums[0] <= plan.phase_node_nums[0] and offs == [0, nums[0]]
    assert all(q <= max(cap, q_tile) for q in wide_q)
    # no two neighbours left that could still be joined
    for v in range(1, nums[0]):
        same = lists[0][v] == lists[0][v - 1] and lists[1][v] == lists[1][v - 1] and lists[2][v - 1] + lists[3][v - 1] == lists[2][v]
        assert not (same and lists[3][v - 1] + lists[3][v] <= cap)
    if name == "c3":
        # 100 root tiles of 16 requests in 4 splits -> 13 per split; 10 x (16, 16, 8) -> 10 x (32, 8)
        assert plan.phase_node_nums[0] == 130 and nums[0] == 4 * 13 + 10 * 2
    # with the kv heads given and no more blocks than compute units, nothing is joined
    *_, nums_few, _ = vnodes_in_launch_order(
        plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
        plan.phase_node_nums, plan.phase_node_offsets, group, 1, light_work=0, q_tile=q_tile)
    if 2 * plan.phase_node_nums[0] * chunks <= 512:
        assert nums_few == list(plan.phase_node_nums)


def _joined_plan(plan, group, hkv, min_blocks):
    """`plan` with its vnode and per-request lists replaced by what join_kv_chunks returns."""
    import copy
    from fasttree_hip.planner import join_kv_chunks
    out = join_kv_chunks(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
                         plan.vnode_to_q_entries, plan.req_to_vnode_entries, plan.req_to_vnode_offs, plan.req_to_vnode_lens,
                         plan.phase_node_nums, plan.phase_node_offsets, group, hkv, min_blocks=min_blocks)
    new = copy.copy(plan)
    (new.vnode_to_kv_offs, new.vnode_to_kv_lens, new.vnode_to_q_offs, new.vnode_to_q_lens,
     new.req_to_vnode_entries, new.req_to_vnode_offs, new.req_to_vnode_lens) = (x.tolist() for x in out[:7])
    new.phase_node_nums, new.phase_node_offsets = out[7], out[8]
    return new


def _attended(plan, batch):
    """For each request: the KV index entries the scratch rows *listed for it* attend."""
    row_vnode = {}
    for v, (qo, ql) in enumerate(zip(plan.vnode_to_q_offs, plan.vnode_to_q_lens)):
        for i in range(ql):
            assert qo + i not in row_vnode, "a scratch row belongs to at most one vnode"
            row_vnode[qo + i] = v
    seen = []
    for r in range(batch):
        rows = plan.req_to_vnode_entries[plan.req_to_vnode_offs[r]: plan.req_to_vnode_offs[r] + plan.req_to_vnode_lens[r]]
        assert rows == sorted(set(rows)) and all(plan.vnode_to_q_entries[x] == r for x in rows)
        got = []
        for x in rows:
            v = row_vnode[x]
            got.extend(range(plan.vnode_to_kv_offs[v], plan.vnode_to_kv_offs[v] + plan.vnode_to_kv_lens[v]))
        seen.append(sorted(got))
    assert sorted(row_vnode) == sorted(x for r in range(batch) for x in
                                       plan.req_to_vnode_entries[plan.req_to_vnode_offs[r]: plan.req_to_vnode_offs[r] + plan.req_to_vnode_lens[r]]), \
        "every row of a kept vnode is listed for its request, and no dropped row is"
    return seen


@pytest.mark.parametrize("name", ["kat1", "c3", "c5_seed0", "c5_seed1", "shape07_h32_8", "rand03", "rand17", "rand41"])
def test_joining_kv_chunks_keeps_what_every_request_attends(name):
    """Forced (one block is enough): every chain of chunks is joined; each request still attends
    the same entries of the flat KV list, each once, through the rows listed for it; the joined
    vnodes keep phase and tile widths; the trailing 32 x -1 are there."""
    case = next(c for c in PLANNER_CASES if c["name"] == name)
    tree, ptrs, batch, plan, params, _ = run_planner(case)
    group = case["Hq"] // case["Hkv"]
    before = _attended(plan, batch)
    new = _joined_plan(plan, group, case["Hkv"], min_blocks=1)
    assert _attended(new, batch) == before
    assert new.req_to_vnode_entries[-32:] == [-1] * 32 and len(new.req_to_vnode_entries) == sum(new.req_to_vnode_lens) + 32
    wide = new.phase_node_nums[0]
    assert new.phase_node_offsets == [0, wide] and sum(new.phase_node_nums) == len(new.vnode_to_kv_offs)
    assert all(n > plan.q_tile_sizes[1] for n in new.vnode_to_q_lens[:wide])
    assert all(n <= plan.q_tile_sizes[1] for n in new.vnode_to_q_lens[wide:])
    # nothing left to join: no run (the vnodes over one KV slice) is followed by a run over the same requests in the same tiles
    runs = {}
    for ko, kl, qo, ql in zip(new.vnode_to_kv_offs, new.vnode_to_kv_lens, new.vnode_to_q_offs, new.vnode_to_q_lens):
        runs.setdefault((ko, kl), []).append(tuple(new.vnode_to_q_entries[qo: qo + ql]))
    for (ko, kl), tiles in runs.items():
        for (ko2, kl2), tiles2 in runs.items():
            assert not (ko2 == ko + kl and tiles2 == tiles)
    if name == "c3":
        # the root's four chunks become one per query tile: 100 + 30 -> 25 + 30 first-phase vnodes, 3 rows fewer per request
        assert plan.phase_node_nums == [130, 400] and new.phase_node_nums == [55, 400]
        assert set(new.req_to_vnode_lens) == {3} and set(plan.req_to_vnode_lens) == {6}
    # the inputs are untouched; with the default thresholds small trees stay as they are, and C3's root gets three
    # chunks of 1344, 1344 and 1312 tokens instead of four (3 x 104 + 160 = 472 first-phase blocks instead of 576)
    same = _joined_plan(plan, group, case["Hkv"], min_blocks=None)
    assert _attended(same, batch) == before
    if name == "c3":
        assert same.phase_node_nums == [3 * 25 + 30, 400] and set(same.req_to_vnode_lens) == {5}
        assert sorted(set(same.vnode_to_kv_lens[:75])) == [1312, 1344] and same.vnode_to_kv_offs[50] == 2688
    elif name not in ("c5_seed0", "c5_seed1"):
        assert same.vnode_to_kv_lens == list(plan.vnode_to_kv_lens) and same.req_to_vnode_entries == list(plan.req_to_vnode_entries)


def test_kv_chunks_are_cut_anew_to_fit_the_first_phase_into_the_machine():
    """C3 (root: 104 blocks per chunk, four chunks; the level below: 160 blocks): the root is cut
    at the shortest chunk length that brings the first phase under the number of resident
    blocks, as long as its own blocks still number nine tenths of `min_blocks`; else it keeps its four chunks."""
    from fasttree_hip.planner import join_kv_chunks
    case = next(c for c in PLANNER_CASES if c["name"] == "c3")
    tree, ptrs, batch, plan, params, _ = run_planner(case)
    before = _attended(plan, batch)
    expectations = [(None, 10**9, 4), (None, 576, 4), (None, 575, 3), (None, 472, 3), (None, 471, 4),  # two chunks: 208 blocks < 230 = 9/10 x 256
                    (232, 471, 2), (233, 471, 4), (105, 368, 2), (105, 367, 1), (105, 264, 1), (105, 263, 4),
                    (104, 10**9, 1)]                                                                   # (104: the root alone fills the machine)
    for min_blocks, resident, chunks in expectations:
        out = join_kv_chunks(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens,
                             plan.vnode_to_q_entries, plan.req_to_vnode_entries, plan.req_to_vnode_offs, plan.req_to_vnode_lens,
                             plan.phase_node_nums, plan.phase_node_offsets, 4, 8, min_blocks=min_blocks, resident_blocks=resident)
        assert out[7] == [25 * chunks + 30, 400], (min_blocks, resident, out[7])
        assert set(out[6].tolist()) == {chunks + 2}
        root = sorted(set(zip(out[0][:25 * chunks].tolist(), out[1][:25 * chunks].tolist())))
        assert len(root) == chunks and root[0][0] == 0 and sum(n for _, n in root) == 4000
        assert all(a + n == b for (a, n), (b, _) in zip(root, root[1:])) and all(n % 64 == 0 for _, n in root[:-1])
    new = _joined_plan(plan, 4, 8, None)
    assert _attended(new, batch) == before


def test_many_equal_chains_are_not_cut_into_a_few_long_blocks():
    """16 nodes of 1500 tokens under a 3000-token root that the planner merges into them: 16
    runs of 4500 tokens in five chunks, 8 blocks per chunk -- 640 blocks.  No run covers the
    machine by itself, so none is cut anew (one chunk of 4500 tokens for some of them would be
    what the launch waits for)."""
    from fasttree_hip.planner import FastTreeParams, fasttree_plan
    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": [1, 16, 256], "lens": [3000, 1500, 100]})
    p = FastTreeParams(); p.set_values(0.66, 0.33, 0.1); p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(4)
    plan = fasttree_plan(tree, ptrs, batch, 8, [1024, 256], [256, 1024], [256, 256], p)
    assert plan.phase_node_nums == [80, 256] and max(plan.vnode_to_kv_lens) == 1024
    new = _joined_plan(plan, 4, 8, None)
    assert new.phase_node_nums == [80, 256] and new.vnode_to_kv_lens == list(plan.vnode_to_kv_lens)


def test_joining_kv_chunks_only_where_the_rows_fill_the_machine():
    """1 x 2048 shared tokens under 1024 requests, 32/8 heads: 4096 query rows = 32 blocks x 8 kv
    heads = 256 blocks without the split, so the root's two chunks are joined; under 256 requests
    (64 blocks) they are not."""
    from fasttree_hip.planner import FastTreeParams, fasttree_plan
    for leaves, joins in ((1024, True), (256, False)):
        tree, ptrs, batch = build_tree({"kind": "regular", "sizes": [1, leaves], "lens": [2048, 32]})
        p = FastTreeParams(); p.set_values(0.66, 0.33, 0.1); p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(4)
        plan = fasttree_plan(tree, ptrs, batch, 8, [1024, 256], [256, 1024], [256, 256], p)
        assert plan.phase_node_nums == [2 * leaves // 16, leaves] and set(plan.req_to_vnode_lens) == {3}
        new = _joined_plan(plan, 4, 8, None)
        if joins:
            assert new.phase_node_nums == [leaves // 16, leaves] and set(new.req_to_vnode_lens) == {2}
            assert set(new.vnode_to_kv_lens[:leaves // 16]) == {2048}
        else:
            assert new.phase_node_nums == plan.phase_node_nums and new.vnode_to_kv_lens == list(plan.vnode_to_kv_lens)
        assert _attended(new, batch) == _attended(plan, batch)


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
