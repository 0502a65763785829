"""Case tables shared by the fixture writer (make_goldens.py) and the tests that read the
fixtures: which trees, head configurations and planner arguments the goldens cover and
how their inputs are rebuilt from seeds.  Pure data plus this repository's own
generators; nothing here touches the reference.
"""

from __future__ import annotations

import hashlib
import random

import numpy as np

from fasttree_hip.kv_tree import (
    assign_requests, generate_irregular_tree, generate_tree, kv_prefix_sums, nodes_from_rows,
)

# The 15 (nodes per level, context per level) shapes the reference sweeps
# (kernel_bench/run_benchmark.sh:5-21) and its three head configurations (:23-27).
BENCH_SHAPES = [
    ([1, 2, 64], [8, 256, 32]),
    ([1, 4, 256], [8, 256, 32]),
    ([1, 4, 8, 256], [8, 256, 256, 32]),
    ([1, 256], [256, 32]),
    ([1, 1024], [2048, 32]),
    ([1, 16, 64], [1024, 256, 32]),
    ([1, 4, 16, 512], [1024, 256, 128, 32]),
    ([1, 4, 16, 64, 256, 1024], [256, 8, 256, 64, 32, 256]),
    ([1, 10], [4000, 400]),
    ([1, 2, 4, 8, 16, 32, 64, 128, 1024], [16] * 9),
    ([1, 2, 4, 8, 16, 32, 64, 128, 1024], [256, 128, 64, 16, 16, 16, 16, 16, 16]),
    ([1, 8, 16, 32, 64, 128, 1024], [256, 128, 64, 16, 16, 16, 16]),
    ([1, 8, 16, 32, 64, 256, 1024], [256, 128, 64, 16, 16, 16, 16]),
    ([1, 16, 32, 64, 128, 1024], [256, 128, 64, 16, 16, 16]),
    ([1, 16, 32, 64, 256, 1024], [256, 128, 64, 16, 16, 16]),
]
BENCH_HEADS = [(16, 1), (32, 8), (32, 32)]


def q_tiles_for_group(g: int):
    """GQA ratio -> query tile sizes: kernel_bench/run_benchmark.sh:46-53 for g in
    {1, 4, 16}; the plugin's rule (64 // g, 16 // g) for the rest (metadata.py:33-34)."""
    return [max(1, 64 // g), max(1, 16 // g)]


def _case(name, tree, Hq, Hkv, D=128, alpha=0.66, beta=0.33, gamma=0.1, TSQs=None, TSKs=(32, 32),
          kv_split_sizes=(1024, 128), para_threshs1=(132, 528), para_threshs2=(132, 132), **extra):
    g = Hq // Hkv
    rec = dict(
        name=name, tree=tree, Hq=Hq, Hkv=Hkv, D=D, alpha=alpha, beta=beta, gamma=gamma,
        TSQs=list(TSQs) if TSQs is not None else q_tiles_for_group(g), TSKs=list(TSKs),
        kv_split_sizes=list(kv_split_sizes), para_threshs1=list(para_threshs1),
        para_threshs2=list(para_threshs2),
    )
    rec.update(extra)
    return rec


def regular(sizes, lens):
    return {"kind": "regular", "sizes": list(sizes), "lens": list(lens)}


def irregular(seed, **kw):
    rec = {"kind": "irregular", "seed": seed}
    rec.update(kw)
    return rec


def random_small_tree(seed: int):
    """Random-parent tree of 2..40 nodes with short runs (rows format)."""
    rng = random.Random(10_000 + seed)
    n = rng.randint(2, 40)
    rows = [[-1, 0, rng.randint(1, 300), 0]]
    for i in range(1, n):
        parent = rng.randint(max(0, i - 6), i - 1)
        rows[parent][3] += 1
        rows.append([parent, i, rng.randint(1, 300), 0])
    return {"kind": "rows", "rows": rows}


def build_tree(spec):
    if spec["kind"] == "regular":
        rows = generate_tree(spec["sizes"], spec["lens"])
    elif spec["kind"] == "irregular":
        kw = {k: v for k, v in spec.items() if k not in ("kind", "seed")}
        rows = generate_irregular_tree(spec["seed"], **kw)
    else:
        rows = spec["rows"]
    tree = nodes_from_rows(rows)
    batch = assign_requests(tree)
    return tree, kv_prefix_sums(tree), batch


def make_params_kwargs(case):
    return dict(alpha=case["alpha"], beta=case["beta"], gamma=case["gamma"], TSQs=case["TSQs"],
                TSKs=case["TSKs"], kv_group_num=case["Hq"] // case["Hkv"])


def digest(arr) -> str:
    return hashlib.sha256(np.ascontiguousarray(arr).tobytes()).hexdigest()


def _planner_cases():
    cases = [
        _case("kat1", regular([1, 1, 2], [100, 50, 10]), 32, 32),
        _case("c1", regular([1, 16], [1024, 128]), 32, 32),
        _case("c2", regular([1, 64], [4096, 256]), 32, 8),
        _case("c3", regular([1, 10, 400], [4000, 400, 40]), 32, 8),
        _case("c4", regular([1, 2048], [512, 1024]), 32, 8),
        # the same trees with thresholds sized for 256 compute units instead of 132
        _case("c2_cu256", regular([1, 64], [4096, 256]), 32, 8, para_threshs1=(256, 1024), para_threshs2=(256, 256)),
        _case("c3_cu256", regular([1, 10, 400], [4000, 400, 40]), 32, 8, para_threshs1=(256, 1024), para_threshs2=(256, 256)),
        _case("c3_q64", regular([1, 10, 400], [4000, 400, 40]), 32, 8, TSQs=(64, 4),
              para_threshs1=(256, 1024), para_threshs2=(256, 256)),
        _case("c4_cu256", regular([1, 2048], [512, 1024]), 32, 8, para_threshs1=(256, 1024), para_threshs2=(256, 256)),
    ]
    for seed in range(3):
        cases.append(_case(f"c5_seed{seed}", irregular(seed), 64, 8))
    for k, (sizes, lens) in enumerate(BENCH_SHAPES):
        for hq, hkv in BENCH_HEADS:
            tag = f"shape{k:02d}_h{hq}_{hkv}"
            cases.append(_case(tag, regular(sizes, lens), hq, hkv))
            # ablations of kernel_bench/run_benchmark.sh:67-81
            cases.append(_case(tag + "_gamma10", regular(sizes, lens), hq, hkv, alpha=0.0, beta=0.0, gamma=10.0,
                               kv_split_sizes=(81920, 81920)))
            cases.append(_case(tag + "_gammam10", regular(sizes, lens), hq, hkv, alpha=0.0, beta=0.0, gamma=-10.0))
    # random small trees with random cost-model parameters (near ties, all loop branches)
    for seed in range(60):
        rng = random.Random(77_000 + seed)
        hq, hkv = rng.choice([(32, 32), (32, 8), (16, 1), (64, 8), (8, 2)])
        g = hq // hkv
        tsq0 = rng.choice([4, 8, 16, 64])
        tsq1 = rng.choice([t for t in (1, 2, 4, 16) if t <= tsq0])
        cases.append(_case(
            f"rand{seed:02d}", random_small_tree(seed), hq, hkv, D=64,
            alpha=round(rng.uniform(0, 1), 2), beta=round(rng.uniform(0, 1), 2),
            gamma=round(rng.uniform(-0.5, 3), 2), TSQs=(tsq0, tsq1),
            TSKs=(rng.choice([16, 32, 64]), rng.choice([16, 32, 128])),
            kv_split_sizes=(rng.choice([64, 256, 1024]), rng.choice([16, 32, 128])),
            para_threshs1=(rng.choice([8, 132, 256]), rng.choice([64, 528, 1024])),
            para_threshs2=(rng.choice([8, 132, 256]), rng.choice([64, 132, 528])),
        ))
    return cases


PLANNER_CASES = _planner_cases()


def _kernel_cases():
    """Small enough for Triton's CPU interpreter to finish in minutes.  TSQs are chosen so
    the planner's adaptation leaves them unchanged (the bench hands its original tile
    lists to the kernel, kernel_bench/benchmark.py:121-122).  All cases are fp16: the
    interpreter has no bfloat16 arithmetic (it computes on the raw bit patterns), so bf16
    is checked against the dense fp64 identity instead."""
    big = dict(para_threshs1=(1, 1), para_threshs2=(1, 1))  # never adapt
    return [
        _case("k_kat1_mha", regular([1, 1, 2], [100, 50, 10]), 4, 4, D=64, dtype="fp16", seed=11, **big),
        _case("k_two_level_gqa4", regular([1, 6], [200, 37]), 8, 2, D=128, dtype="fp16", seed=12, **big),
        _case("k_three_level_gqa4", regular([1, 3, 24], [150, 70, 19]), 8, 2, D=128, dtype="fp16", seed=13,
              kv_split_sizes=(64, 32), **big),
        _case("k_irregular_gqa8", irregular(5, levels=4, fanout_range=(1, 4), len_range=(4, 90), max_leaves=40),
              16, 2, D=128, dtype="fp16", seed=15, kv_split_sizes=(128, 32), **big),
        _case("k_mha_d32", regular([1, 20], [96, 8]), 2, 2, D=32, dtype="fp16", seed=16, **big),
        _case("k_all_merge", regular([1, 4, 8], [60, 30, 10]), 8, 2, D=128, dtype="fp16", seed=17,
              alpha=0.0, beta=0.0, gamma=10.0, kv_split_sizes=(81920, 81920), **big),
        # C1 of the baseline in full: 32/32 heads, root 1024 tokens, 16 leaves of 128
        _case("k_c1", regular([1, 16], [1024, 128]), 32, 32, D=128, dtype="fp16", seed=18),
        # C2 and C3 of the baseline at full size; the fixtures keep the outputs of every
        # `keep_every`-th request only (the interpreter still runs the whole launch)
        dict(_case("k_c2", regular([1, 64], [4096, 256]), 32, 8, D=128, dtype="fp16", seed=19, **big), keep_every=4),
        dict(_case("k_c3", regular([1, 10, 400], [4000, 400, 40]), 32, 8, D=128, dtype="fp16", seed=20, **big),
             keep_every=16),
    ]


KERNEL_CASES = _kernel_cases()


def kernel_case_inputs(case, tree, ptrs, batch):
    """Q [B,Hq,D], K/V [T,Hkv,D] for a kernel case, node-major pool, as CPU torch tensors."""
    import torch

    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16}[case["dtype"]]
    rng = np.random.default_rng(case["seed"])
    total = ptrs[-1]

    def draw(shape):
        return torch.from_numpy(rng.standard_normal(shape, dtype=np.float32)).to(dtype)

    k = draw((total, case["Hkv"], case["D"]))
    v = draw((total, case["Hkv"], case["D"]))
    q = draw((batch, case["Hq"], case["D"]))
    return q, k, v


def _deft_cases():
    """Trees for the comparison engine (DeFT-Flatten): subtrees that span several nodes and nodes
    that span several subtrees, query sets of more than one mask word (more than 64 requests) and
    of more than one pass of a thread block (more than 128 query rows), MHA and GQA.  ``q_tile``
    is the reference kernel's Q_TILE_SIZE (a divisor of mask_len)."""
    def case(name, tree, hq, hkv, d, seed, subtree_len=128, mask_len=64, q_tile=16):
        return dict(name=name, tree=tree, Hq=hq, Hkv=hkv, D=d, dtype="fp16", seed=seed, subtree_len=subtree_len,
                    mask_len=mask_len, q_tile=q_tile)
    return [
        case("kat1_mha", regular([1, 1, 2], [100, 50, 10]), 4, 4, 64, 31, subtree_len=32),
        case("two_level_gqa4", regular([1, 6], [200, 37]), 8, 2, 128, 32),
        case("three_level_gqa4", regular([1, 3, 24], [150, 70, 19]), 8, 2, 128, 33),
        case("irregular_gqa8", irregular(5, levels=4, fanout_range=(1, 4), len_range=(4, 90), max_leaves=40), 16, 2, 128, 35),
        case("many_requests_gqa4", regular([1, 2, 70], [50, 30, 7]), 8, 2, 64, 36, subtree_len=64),
        case("mha_d32_two_words", regular([1, 90], [40, 5]), 2, 2, 32, 37),
    ]


DEFT_CASES = _deft_cases()


def gathered_cache(tree, ptrs, k_pool, v_pool):
    """The per-request gathered, zero-padded caches ``[B, max_seqlen, Hkv, D]`` of
    kernel_bench/flash_attn_wrap.py:36-67 from a node-major pool (CPU tensors)."""
    import torch

    paths = {}
    for index, node in enumerate(tree):
        if node.num_children == 0:
            chain, cur = [], index
            while cur >= 0:
                chain.append(cur)
                cur = tree[cur].parent
            for r in node.requests:
                paths[r] = list(reversed(chain))
    batch = len(paths)
    tokens = [np.concatenate([np.arange(ptrs[n], ptrs[n + 1]) for n in paths[r]]) for r in range(batch)]
    width = max(len(t) for t in tokens)
    k_cache = torch.zeros((batch, width) + tuple(k_pool.shape[1:]), dtype=k_pool.dtype)
    v_cache = torch.zeros_like(k_cache)
    for r, t in enumerate(tokens):
        idx = torch.from_numpy(t.astype(np.int64))
        k_cache[r, : len(t)] = k_pool[idx]
        v_cache[r, : len(t)] = v_pool[idx]
    return k_cache, v_cache
