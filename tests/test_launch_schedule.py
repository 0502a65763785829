"""The launch schedule of the first decode stage (block programs), on the CPU: whatever the
arrangement, every request attends every token of its path exactly once, through scratch rows
that are listed for it; the program table describes the lists it comes with."""

import numpy as np
import pytest

from cases import PLANNER_CASES, build_tree
from fasttree_hip import launch_schedule as ls
from fasttree_hip.launch_schedule import LaunchPhases, block_programs
from helpers import run_planner

NAMES = ["kat1", "c1", "c3", "c5_seed0", "c5_seed1", "shape07_h32_8", "shape07_h16_1_gamma10", "rand03", "rand17", "rand41"]
VARIANTS = {
    "default": {},
    "cut_anew": dict(recut=True),
    "planner_chunks": dict(recut=False),
    "narrow_in_programs": dict(recut=True, embed=True),
    "narrow_in_programs_auto": dict(embed=None),
    "one_block_per_unit": dict(block_slots=256),
    "two_blocks_per_unit": dict(block_slots=512, recut=True),
    "packed": dict(layout="packed"),
    "resident": dict(layout="resident"),
}


def _attended(kv_offs, kv_lens, q_offs, q_lens, q_entries, req_entries, req_offs, req_lens, batch):
    """For each request: the KV index entries the scratch rows *listed for it* attend."""
    row_vnode = {}
    for v, (qo, ql) in enumerate(zip(q_offs, q_lens)):
        for i in range(ql):
            assert qo + i not in row_vnode, "a scratch row belongs to at most one vnode"
            row_vnode[qo + i] = v
    assert sorted(row_vnode) == list(range(len(q_entries))), "every scratch row belongs to a vnode"
    seen = []
    for r in range(batch):
        rows = list(req_entries[req_offs[r]: req_offs[r] + req_lens[r]])
        assert rows == sorted(set(rows)) and all(q_entries[x] == r for x in rows)
        got = []
        for x in rows:
            v = row_vnode[x]
            got.extend(range(kv_offs[v], kv_offs[v] + kv_lens[v]))
        seen.append(sorted(got))
    assert sum(req_lens[:batch]) == len(q_entries), "every scratch row is listed for its request"
    return seen


def _plan_lists(plan):
    return (plan.vnode_to_kv_offs, plan.vnode_to_kv_lens, plan.vnode_to_q_offs, plan.vnode_to_q_lens, plan.vnode_to_q_entries)


def _schedule(case, **kw):
    tree, ptrs, batch, plan, params, _ = run_planner(case)
    group = case["Hq"] // case["Hkv"]
    sched = block_programs(*_plan_lists(plan), batch, group, case["Hkv"], **kw)
    return plan, batch, group, sched


@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("name", NAMES)
def test_every_request_still_attends_its_path_once(name, variant):
    case = next(c for c in PLANNER_CASES if c["name"] == name)
    plan, batch, group, s = _schedule(case, **VARIANTS[variant])
    before = _attended(*_plan_lists(plan), plan.req_to_vnode_entries, plan.req_to_vnode_offs, plan.req_to_vnode_lens, batch)
    after = _attended(s.kv_offs.tolist(), s.kv_lens.tolist(), s.q_offs.tolist(), s.q_lens.tolist(), s.q_entries.tolist(),
                      s.req_entries.tolist(), s.req_offs.tolist(), s.req_lens.tolist(), batch)
    assert after == before
    # the per-request lists end with the reference's padding (kernel_bench/fasttree.py:261-262)
    assert s.req_entries[-32:].tolist() == [-1] * 32 and len(s.req_entries) == s.num_rows + 32
    # phases: the programs' vnodes first, then the vnodes served one wave each
    n_wide, n_narrow = s.phase_node_nums
    assert s.phase_node_offsets == [0, n_wide] and n_wide + n_narrow == len(s.kv_offs)
    assert (s.q_lens[:n_wide] * group <= ls.BLOCK_ROWS).all(), "a program's vnode fits one pass of a block"
    assert (s.kv_lens > 0).all()


@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("name", NAMES)
def test_program_table_describes_the_lists(name, variant):
    case = next(c for c in PLANNER_CASES if c["name"] == name)
    _, _, _, s = _schedule(case, **VARIANTS[variant])
    t = s.prog_table
    n_wide, n_narrow = s.phase_node_nums
    assert t.shape == (s.num_programs, 4) and t.dtype == np.int32
    if n_wide == 0:
        assert s.num_programs == 0 and s.narrow_in_programs == 0
        return
    # every wide vnode belongs to exactly one program, in order, and no program is empty
    assert t[0, 0] == 0 and t[-1, 1] == n_wide
    assert (t[1:, 0] == t[:-1, 1]).all() and (t[:, 1] > t[:, 0]).all()
    # the programs' narrow vnodes lie back to back at the head of the second phase
    counts = np.abs(t[:, 3])
    assert (t[:, 2] == np.concatenate([[0], np.cumsum(counts)[:-1]])).all()
    assert counts.sum() == s.narrow_in_programs <= n_narrow
    if not VARIANTS[variant].get("embed", False):
        assert s.narrow_in_programs == 0 or VARIANTS[variant].get("embed", False) is None
    assert len(s.program_tiles) == s.num_programs and (s.program_tiles > 0).all()
    assert s.modelled_us > 0


def test_headline_tree_is_cut_into_equal_programs():
    """C3 (3-level tree, 400 requests, 32/8 heads): the 4000-token root under 1600 query rows and
    the ten 400-token nodes under 160 rows become at most 64 programs per kv head (512 block
    slots / 8 heads) whose modelled work differs by a few percent; pieces start and end at
    multiples of 64 tokens of their run; the 400 leaves stay as the planner made them."""
    case = next(c for c in PLANNER_CASES if c["name"] == "c3")
    plan, batch, group, s = _schedule(case, block_slots=512, layout="packed")
    assert 56 <= s.num_programs <= 64
    assert s.program_tiles.max() <= 1.1 * s.program_tiles.mean()
    n_wide, n_narrow = s.phase_node_nums
    assert n_narrow == 400 and sorted(s.kv_lens[n_wide:].tolist()) == [40] * 400 and set(s.q_lens[n_wide:].tolist()) == {1}
    root = [(int(o), int(n)) for o, n in zip(s.kv_offs[:n_wide], s.kv_lens[:n_wide]) if o < 4000]
    assert all(o % ls.CUT_TOKENS == 0 for o, _ in root) and all(n >= ls.MIN_PIECE_TOKENS for _, n in root)
    # every row chunk of the root covers its 4000 tokens once
    by_rows = {}
    for v in range(n_wide):
        if s.kv_offs[v] < 4000:
            by_rows.setdefault(int(s.q_entries[s.q_offs[v]]), []).append((int(s.kv_offs[v]), int(s.kv_lens[v])))
    assert len(by_rows) == 13   # 1600 rows in 13 even chunks of at most 128
    for pieces in by_rows.values():
        pieces.sort()
        assert pieces[0][0] == 0 and sum(n for _, n in pieces) == 4000
        assert all(a + n == b for (a, n), (b, _) in zip(pieces, pieces[1:]))


def test_headline_tree_gets_a_block_per_piece_when_all_fit():
    """C3 by default: every (run, row chunk) has programs of its own, all resident from the start
    (at most 64 per kv head).  The root is cut into as many equal pieces as still fit -- three,
    at the same multiples of 64 tokens for all 13 row chunks, one of them shorter (the pieces that
    end up as the younger block of a compute unit) -- the ten 400-token nodes stay whole, programs are listed longest first, and the modelled duration is within
    RESIDENT_MARGIN of the packed layout's."""
    case = next(c for c in PLANNER_CASES if c["name"] == "c3")
    plan, batch, group, s = _schedule(case)
    packed = _schedule(case, layout="packed")[3]
    assert s.block_slots == 512 and s.num_programs == 13 * 3 + 20 == s.phase_node_nums[0]
    assert (s.prog_table[:, 1] - s.prog_table[:, 0] == 1).all() and (s.prog_table[:, 3] == 0).all()
    assert (np.diff(s.program_tiles) <= 0).all()
    assert s.modelled_us <= ls.RESIDENT_MARGIN * packed.modelled_us
    n_wide = s.phase_node_nums[0]
    root = sorted({(int(o), int(n)) for o, n in zip(s.kv_offs[:n_wide], s.kv_lens[:n_wide]) if o < 4000})
    # three pieces at multiples of 64 tokens, the same for all 13 row chunks; 7 of the 39 have to be
    # the younger block of a compute unit, so one piece per chunk is about SHORT_PIECE_RATIO of the others
    assert root == [(0, 1408), (1408, 1408), (2816, 1184)]
    assert all(o % ls.CUT_TOKENS == 0 for o, _ in root) and sum(n for _, n in root) == 4000
    assert abs(root[2][1] / root[1][1] - ls.SHORT_PIECE_RATIO) < 0.05
    assert s.kv_lens[:26].min() >= 1408 and set(s.kv_lens[26:39].tolist()) == {1184}  # the younger blocks (programs 32..38) are short ones
    rest = sorted({(int(o), int(n)) for o, n in zip(s.kv_offs[:n_wide], s.kv_lens[:n_wide]) if o >= 4000})
    assert rest == [(4000 + 400 * i, 400) for i in range(10)]
    assert s.num_rows == 400 * 5 < packed.num_rows          # three root rows, one node row, one leaf row a request
    # a tree whose wide work items outnumber the programs of a round has no such layout
    c5 = next(c for c in PLANNER_CASES if c["name"] == "c5_seed0")
    a, b = _schedule(c5)[3], _schedule(c5, layout="packed")[3]
    assert a.num_programs == b.num_programs and np.array_equal(a.kv_offs, b.kv_offs)


def test_small_launches_keep_the_planner_chunks():
    """A launch whose programs would hold less than MIN_PROGRAM_TILES keeps the planner's KV
    chunks, one vnode per program, longest first; a launch without wide vnodes has no programs,
    and while its narrow vnodes would leave most wave slots idle its long runs are halved down to
    pieces of 128 tokens (C1: 17 vnodes x 32 heads; the 1024-token root becomes 8 pieces)."""
    case = next(c for c in PLANNER_CASES if c["name"] == "c1")
    plan, batch, group, s = _schedule(case)
    assert s.num_programs == 0 and s.phase_node_nums == [0, 16 + 8]
    want = sorted((o, n) for o, n in zip(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens) if n != 1024) + []
    root = [(o, n) for o, n in zip(plan.vnode_to_kv_offs, plan.vnode_to_kv_lens) if n == 1024]
    assert len(root) == 1
    want += [(root[0][0] + 128 * i, 128) for i in range(8)]
    assert sorted(zip(s.kv_offs.tolist(), s.kv_lens.tolist())) == sorted(want)
    assert s.num_rows == 16 + 8 * 16 and s.req_lens.tolist() == [9] * 16
    # a launch that fills the wave slots keeps its runs whole
    full = ls._cut_long_narrow_runs([(1000 * i, 600, [i]) for i in range(300)], 1, 8, 2048)
    assert len(full) == 300
    some = ls._cut_long_narrow_runs([(0, 600, [0, 1]), (600, 100, [2])], 4, 8, 2048)
    assert sorted((o, n) for o, n, _ in some) == [(0, 160), (160, 160), (320, 280), (600, 100)]
    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": [1, 64], "lens": [512, 32]})
    from fasttree_hip.planner import FastTreeParams, fasttree_plan
    p = FastTreeParams(); p.set_values(0.66, 0.33, 0.1); p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(4)
    plan = fasttree_plan(tree, ptrs, batch, 8, [256, 256], [1, 1], [1, 1], p)
    assert plan.phase_node_nums[0] == 8
    s = block_programs(*_plan_lists(plan), batch, 4, 8)
    n_wide = s.phase_node_nums[0]
    assert s.num_programs == n_wide > 0 and (s.prog_table[:, 1] - s.prog_table[:, 0] == 1).all()
    chunk_lens = sorted(set(plan.vnode_to_kv_lens[: plan.phase_node_nums[0]]))
    assert sorted(set(s.kv_lens[:n_wide].tolist())) == chunk_lens
    assert (np.diff(s.program_tiles) <= 0).all()


def test_narrow_vnodes_dealt_to_programs_in_equal_shares():
    """With embed=True every program gets its share of the narrow vnodes (counts differ by at
    most one), the two halves of a round of programs in opposite orders (negative count: before
    the wide vnodes)."""
    case = next(c for c in PLANNER_CASES if c["name"] == "c3")
    _, _, _, s = _schedule(case, recut=True, embed=True, block_slots=512)
    counts = np.abs(s.prog_table[:, 3])
    assert s.narrow_in_programs == 400 == counts.sum() and counts.max() - counts.min() <= 1
    per_round = 512 // 8
    front = s.prog_table[:, 3] < 0
    assert front[: per_round // 2].all() and not front[per_round // 2: per_round].any()


def test_preparation_in_launch_order_carries_the_programs():
    """fasttree_preparation(launch_order=True): the phase list is a list of two counts that also
    carries the program table (a device tensor) -- with and without preallocated buffers."""
    import torch
    from fasttree_hip.planner import FastTreeParams, PlanBuffers, fasttree_preparation
    case = next(c for c in PLANNER_CASES if c["name"] == "c3")
    tree, ptrs, batch = build_tree(case["tree"])
    buffers = PlanBuffers(32, 128, max_kv_entries=400000, max_rows=8192, max_vnodes=8192, max_batch_size=2048, device="cpu")
    outs = []
    for buf in (None, buffers):
        p = FastTreeParams(); p.set_values(0.66, 0.33, 0.1); p.set_q_tile_sizes([16, 4]); p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(4)
        aux, _ = fasttree_preparation(tree, ptrs, batch, 32, 8, 128, [1024, 256], [256, 1024], [256, 256], p,
                                      device="cpu", launch_order=True, buffers=buf)
        nums = aux[11]
        assert isinstance(nums, LaunchPhases) and isinstance(nums, list) and len(nums) == 2 and aux[12] == [0, nums[0]]
        assert nums.prog_table.dtype == torch.int32 and nums.prog_table.numel() == 4 * nums.num_programs > 0
        assert int(nums.prog_table.view(-1, 4)[-1, 1]) == nums[0] and nums.narrow_in_programs == 0
        assert aux[9].shape[0] == aux[3].numel() == int(aux[8].sum())
        outs.append(aux)
    for a, b in zip(outs[0][:9], outs[1][:9]):
        assert torch.equal(a, b)
    assert torch.equal(outs[0][11].prog_table, outs[1][11].prog_table)
    assert outs[1][11].prog_table.data_ptr() == buffers.prog_table.data_ptr()


@pytest.mark.parametrize("kw", [dict(), dict(recut=True), dict(recut=True, layout="packed"), dict(recut=False)])
def test_a_shared_run_without_tokens_is_scheduled(kw):
    """A node of zero tokens shared by many requests (more than 16 query rows: a wide run with no
    tile steps) is arranged like any other: it gets scratch rows, which the kernels fill with empty
    partial results, and no program is built from nothing."""
    reqs = 40
    # vnode 0: the empty shared root; vnode 1: a shared run of 300 tokens; then one leaf per request
    kv_offs = [0, 0] + [300 + 20 * r for r in range(reqs)]
    kv_lens = [0, 300] + [20] * reqs
    q_offs = [0, reqs] + [2 * reqs + r for r in range(reqs)]
    q_lens = [reqs, reqs] + [1] * reqs
    q_entries = list(range(reqs)) * 2 + list(range(reqs))
    sched = block_programs(kv_offs, kv_lens, q_offs, q_lens, q_entries, reqs, 4, 8, **kw)
    seen = _attended(sched.kv_offs, sched.kv_lens, sched.q_offs, sched.q_lens, sched.q_entries,
                     sched.req_entries, sched.req_offs, sched.req_lens, reqs)
    for r in range(reqs):
        assert seen[r] == sorted(list(range(300)) + list(range(300 + 20 * r, 320 + 20 * r)))
    # only the empty root everywhere: nothing to cut, nothing to fail on
    alone = block_programs([0], [0], [0], [reqs], list(range(reqs)), reqs, 4, 8, **kw)
    assert alone.num_rows == reqs and int(alone.kv_lens.sum()) == 0


@pytest.mark.parametrize("num_cus", [128, 256, 304])
@pytest.mark.parametrize("name", ["c3", "c5_seed0", "shape07_h32_8"])
def test_layout_follows_the_number_of_compute_units(name, num_cus):
    """The programs are laid out for the device's compute units, not for a fixed machine: on 128
    units (a partitioned or smaller part) and on 304 (an MI300X) the same plan gives a schedule
    with the same coverage whose programs of one round fit that machine's block slots -- two per
    unit, or one per unit where that layout's modelled duration is the shorter."""
    case = next(c for c in PLANNER_CASES if c["name"] == name)
    plan, batch, group, s = _schedule(case, num_cus=num_cus)
    assert s.num_cus == num_cus and s.block_slots in (num_cus, 2 * num_cus)
    want = _attended(*_plan_lists(plan), plan.req_to_vnode_entries, plan.req_to_vnode_offs, plan.req_to_vnode_lens, batch)
    got = _attended(s.kv_offs, s.kv_lens, s.q_offs, s.q_lens, s.q_entries, s.req_entries, s.req_offs, s.req_lens, batch)
    assert got == want
    heads = case["Hkv"]
    rounds = max(1, int(np.ceil(s.program_tiles.sum() / ((s.block_slots // heads) * ls.MAX_PROGRAM_TILES)))) if s.num_programs else 1
    assert s.num_programs <= max(1, s.block_slots // heads) * rounds or s.num_programs == s.phase_node_nums[0]


def test_fewer_compute_units_mean_fewer_and_longer_programs():
    case = next(c for c in PLANNER_CASES if c["name"] == "c3")
    small = _schedule(case, num_cus=128, layout="packed")[3]
    full = _schedule(case, num_cus=256, layout="packed")[3]
    large = _schedule(case, num_cus=304, layout="packed")[3]
    assert small.num_programs < full.num_programs <= large.num_programs
    assert small.program_tiles.max() > full.program_tiles.max() >= large.program_tiles.max()
    assert small.modelled_us > full.modelled_us >= large.modelled_us
    # without a device to ask, the default machine is an MI355X's 256 units
    assert ls.compute_units("cpu") == 256 == ls.DEFAULT_COMPUTE_UNITS


def test_narrow_records_repeat_the_lists(monkeypatch):
    """The record of a narrow vnode holds what the lists say about it: its four entries, the
    requests of its scratch rows and the pool slots of its first 32 tokens, the last one repeated
    past the end of a shorter run (hand case, then every narrow vnode of two launch-order plans)."""
    kv_entries = np.arange(1000, 1100)
    rec = ls.narrow_records(kv_entries, [0, 10, 50], [10, 40, 3], [0, 2, 3], [2, 1, 4], [7, 8, 9, 3, 4, 5, 6], 1, 2)
    assert rec.shape == (2, 64) and rec.dtype == np.int32
    assert rec[0, :4].tolist() == [10, 40, 2, 1] and rec[0, 4] == 9
    assert rec[0, 20:52].tolist() == list(range(1010, 1042))
    assert rec[1, :4].tolist() == [50, 3, 3, 4] and rec[1, 4:8].tolist() == [3, 4, 5, 6]
    assert rec[1, 20:52].tolist() == [1050, 1051] + [1052] * 30
    assert ls.narrow_records(kv_entries, [0], [0], [0], [0], [], 0, 1)[0].tolist() == [0] * 64     # an empty vnode
    import torch
    from fasttree_hip.planner import FastTreeParams, fasttree_preparation
    import fasttree_hip.planner as planner_module
    monkeypatch.setattr(planner_module, "VERBOSE", False)
    for name in ("c3", "c5_seed0", "c1"):
        case = next(c for c in PLANNER_CASES if c["name"] == name)
        tree, ptrs, batch = build_tree(case["tree"])
        g = case["Hq"] // case["Hkv"]
        p = FastTreeParams(); p.set_values(0.66, 0.33, 0.1); p.set_q_tile_sizes([max(1, 64 // g), max(1, 16 // g)])
        p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(g)
        slot_map = np.random.default_rng(0).permutation(ptrs[-1])
        aux, _ = fasttree_preparation(tree, ptrs, batch, case["Hq"], case["Hkv"], 128, [1024, 256], [256, 1024], [256, 256], p,
                                      device="cpu", kv_slot_map=slot_map, launch_order=True)
        nums, offs = aux[11], aux[12]
        table = nums.narrow_table.view(-1, 64).numpy()
        assert table.shape[0] == nums[1] > 0
        kv_entries, kv_offs, kv_lens, q_entries, q_offs, q_lens = (t.numpy() for t in aux[:6])
        for i in range(0, nums[1], max(1, nums[1] // 50)):
            v = offs[1] + i
            assert table[i, :4].tolist() == [kv_offs[v], kv_lens[v], q_offs[v], q_lens[v]]
            assert table[i, 4:4 + min(q_lens[v], 16)].tolist() == q_entries[q_offs[v]: q_offs[v] + min(q_lens[v], 16)].tolist()
            want = [kv_entries[kv_offs[v] + min(t, kv_lens[v] - 1)] for t in range(32)]
            assert table[i, 20:52].tolist() == want
        # the per-request records of the merge launch: length, offset, the first 14 scratch rows
        req_entries, req_offs, req_lens = (t.numpy() for t in aux[6:9])
        records = nums.req_table.view(-1, 16).numpy()
        assert records.shape[0] == batch
        for r in range(0, batch, max(1, batch // 60)):
            n, off = int(req_lens[r]), int(req_offs[r])
            assert records[r, :2].tolist() == [n, off]
            assert records[r, 2:2 + min(n, 14)].tolist() == req_entries[off: off + min(n, 14)].tolist()


def test_program_records_repeat_the_lists(monkeypatch):
    """The record of a block program holds what the lists say about its first wide vnode: the four
    list entries, the requests of its rows, the pool slots of its first 64 tokens (the last one
    repeated past a shorter run); programs without a wide vnode, or with one of more than 128 query
    rows, are flagged as having none (hand case, then the programs of three launch-order plans)."""
    kv_entries = np.arange(500, 800)
    #             vnode:   0    1    2
    kv_offs, kv_lens = [0, 100, 130], [100, 30, 70]
    q_offs, q_lens = [0, 40, 43], [40, 3, 33]
    q_entries = list(range(900, 976))
    table = [[1, 2, 0, 0], [0, 1, 0, 0], [2, 2, 0, 0], [2, 3, 0, 0]]       # programs: vnode 1; vnode 0; none; vnode 2
    rec = ls.program_records(kv_entries, kv_offs, kv_lens, q_offs, q_lens, q_entries, table, 0, 4)
    assert rec.shape == (4, 256) and rec.dtype == np.int32
    assert rec[0, :5].tolist() == [100, 30, 40, 3, 1]
    assert rec[0, 8:11].tolist() == [940, 941, 942]
    assert rec[0, 136:200].tolist() == list(range(600, 630)) + [629] * 34
    assert rec[1, :5].tolist() == [0, 100, 0, 40, 0]                       # 40 requests x 4 heads: more than 128 rows
    assert rec[2, 4] == 0 and rec[3, :5].tolist() == [130, 70, 43, 33, 0]  # no wide vnode; 132 rows
    assert ls.program_records(kv_entries, kv_offs, kv_lens, q_offs, q_lens, q_entries, table, 0, 1)[1, 4] == 1
    assert ls.program_records([], [], [], [], [], [], np.zeros((0, 4)), 0, 4).shape == (0, 256)
    import fasttree_hip.planner as planner_module
    from fasttree_hip.planner import FastTreeParams, fasttree_preparation
    monkeypatch.setattr(planner_module, "VERBOSE", False)
    for name in ("c3", "c5_seed0", "c2"):
        case = next(c for c in PLANNER_CASES if c["name"] == name)
        tree, ptrs, batch = build_tree(case["tree"])
        g = case["Hq"] // case["Hkv"]
        p = FastTreeParams(); p.set_values(0.66, 0.33, 0.1); p.set_q_tile_sizes([max(1, 64 // g), max(1, 16 // g)])
        p.set_kv_tile_sizes([32, 32]); p.set_kv_group_num(g)
        slot_map = np.random.default_rng(0).permutation(ptrs[-1])
        aux, _ = fasttree_preparation(tree, ptrs, batch, case["Hq"], case["Hkv"], 128, [1024, 256], [256, 1024], [256, 256], p,
                                      device="cpu", kv_slot_map=slot_map, launch_order=True)
        nums, offs = aux[11], aux[12]
        records = nums.prog_records.view(-1, 256).numpy()
        programs = nums.prog_table.view(-1, 4).numpy()
        assert records.shape[0] == nums.num_programs == len(programs) > 0
        kv_entries, kv_offs, kv_lens, q_entries, q_offs, q_lens = (t.numpy() for t in aux[:6])
        assert records[:, 4].all()            # every program of these plans starts with a vnode of at most 128 rows
        for i in range(0, len(programs), max(1, len(programs) // 40)):
            v = offs[0] + programs[i, 0]
            assert records[i, :4].tolist() == [kv_offs[v], kv_lens[v], q_offs[v], q_lens[v]]
            assert records[i, 8:8 + q_lens[v]].tolist() == q_entries[q_offs[v]: q_offs[v] + q_lens[v]].tolist()
            assert records[i, 136:200].tolist() == [kv_entries[kv_offs[v] + min(t, kv_lens[v] - 1)] for t in range(64)]


def test_request_records_by_hand():
    rec = ls.request_records([5, 6, 7, 9, 1, 2, 3, -1, -1], [0, 3, 4], [3, 1, 3])
    assert rec.shape == (3, 16) and rec.dtype == np.int32
    assert rec[0].tolist() == [3, 0, 5, 6, 7] + [0] * 11
    assert rec[1].tolist() == [1, 3, 9] + [0] * 13
    assert rec[2].tolist() == [3, 4, 1, 2, 3] + [0] * 11
    long = ls.request_records(list(range(100, 130)), [0, 20], [20, 10])      # more rows than a record holds
    assert long[0].tolist() == [20, 0] + list(range(100, 114))
    assert long[1].tolist() == [10, 20] + list(range(120, 130)) + [0] * 4
    assert ls.request_records([], [], []).shape == (0, 16)
    assert ls.request_records([], [0], [0])[0].tolist() == [0] * 16          # a request without rows


def test_modelled_duration_of_narrow_launches_by_hand():
    """The modelled duration of launches of narrow vnodes alone, worked by hand: ten vnodes of four
    tiles leave the wave slots empty, so four waves share each (one tile step per wave, plus the
    merge of the four); 2000 vnodes of one tile for one kv head fill the slots, one wave each; with
    eight kv heads they take eight rounds' worth of the slots."""
    us = ls.TILE_US_SHARED
    few = ls.block_programs([128 * i for i in range(10)], [128] * 10, list(range(10)), [1] * 10, list(range(10)), 10, 16, 1,
                            num_cus=256)
    assert few.phase_node_nums == [0, 10]
    want = (ls.NARROW_STARTUP_TILES + ls.NARROW_STEP_TILES * 1 + ls.NARROW_SHARE_TILES) * us + ls.LAUNCH_US
    assert few.modelled_us == pytest.approx(want)
    n = 2000
    many = ls.block_programs([32 * i for i in range(n)], [32] * n, list(range(n)), [1] * n, list(range(n)), n, 16, 1, num_cus=256)
    item = (ls.NARROW_STARTUP_TILES + ls.NARROW_STEP_TILES) * us
    stream = n * 32 * 4 * 128 / ls.NARROW_BYTES_PER_US                       # K and V rows of one head at the narrow rate
    assert item < stream < 1.1 * item
    assert many.modelled_us == pytest.approx(stream + ls.LAUNCH_US)          # 2000 waves on 2048 slots: one item, or its bytes
    eight = ls.block_programs([32 * i for i in range(n)], [32] * n, list(range(n)), [1] * n, list(range(n)), n, 4, 8, num_cus=256)
    assert eight.modelled_us == pytest.approx(max(item * n * 8 / 2048, 8 * stream) + ls.LAUNCH_US)
