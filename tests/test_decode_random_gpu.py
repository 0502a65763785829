"""Seeded random trees, head configurations and planner settings on the GPU: the tree decode
against the fp64 dense oracle on sampled requests and against this library's decode over
per-request gathered caches on all of them.  The cases are fixed by their seeds; they are meant
to reach the rarer code paths together (ranking fall-back, row chunks, shared narrow vnodes,
multi-pass narrow vnodes, light first-phase vnodes, both launch orders)."""
import math
import random

import numpy as np
import pytest
import torch

import fasttree_oracle as oracle
from cases import build_tree
from fasttree_hip.decode import fasttree_decode, gathered_decode
from fasttree_hip.inputs import gather_per_request, make_decode_inputs
from fasttree_hip.planner import FastTreeParams, fasttree_preparation
from helpers import arith_reference, assert_like_for_like, assert_parity

pytestmark = pytest.mark.gpu

HEADS = [(8, 8), (16, 4), (32, 8), (16, 1), (64, 8), (32, 32)]


def random_case(seed):
    rng = random.Random(1000 + seed)
    if rng.random() < 0.4:
        spec = {"kind": "irregular", "seed": 100 + seed, "levels": rng.randint(3, 5), "fanout_range": (1, rng.choice([4, 6, 8])),
                "len_range": (rng.choice([1, 8, 16]), rng.choice([200, 600, 1500])), "max_leaves": rng.choice([60, 300, 700])}
    else:
        depth = rng.randint(2, 5)
        sizes, lens = [1], [rng.choice([3, 17, 64, 300, 1500, 2600])]
        for _ in range(depth - 1):
            sizes.append(sizes[-1] * rng.choice([1, 2, 3, 5, 8, 16]))
            lens.append(rng.choice([1, 7, 16, 33, 128, 500]))
        while sizes[-1] > 700:
            sizes[-1] //= 2
        sizes = [max(s, p) for s, p in zip(sizes, [1] + sizes[:-1])]
        spec = {"kind": "regular", "sizes": sizes, "lens": lens}
    hq, hkv = rng.choice(HEADS)
    d = rng.choice([64, 128, 128, 128])
    dtype = rng.choice([torch.float16, torch.float16, torch.bfloat16])
    g = hq // hkv
    q_tiles = rng.choice([[max(1, 64 // g), max(1, 16 // g)], [max(1, 256 // g), max(1, 16 // g)], [max(2, 40 // g), 1]])
    splits = rng.choice([[1024, 128], [256, 64], [4096, 4096], [512, 128]])
    thr = rng.choice([((132, 528), (132, 132)), ((256, 1024), (256, 256)), ((1, 1), (1, 1)), ((10**6, 10**6), (1, 1))])
    abg = rng.choice([(0.66, 0.33, 0.1), (0.66, 0.33, 0.1), (0.0, 0.0, 10.0), (0.0, 0.0, -10.0), (0.2, 0.9, 0.5)])
    return dict(spec=spec, hq=hq, hkv=hkv, d=d, dtype=dtype, q_tiles=q_tiles, splits=splits, thr=thr, abg=abg,
                launch_order=rng.random() < 0.7)


# (seeds 24 and 44 draw pools of more than 2**27 elements and are left out)
@pytest.mark.parametrize("seed", [s for s in range(50) if s not in (24, 44)])
def test_random_tree_and_settings(seed, device):
    c = random_case(seed)
    print("\n[gpu case] random", seed, {k: v for k, v in c.items() if k != "spec"}, c["spec"], flush=True)
    tree, ptrs, batch = build_tree(c["spec"])
    assert ptrs[-1] * c["hkv"] * c["d"] <= (1 << 27), "pool larger than this test is meant for"
    inp = make_decode_inputs(tree, c["hq"], c["hkv"], c["d"], device=device, dtype=c["dtype"], seed=seed, shuffle_slots=True)
    params = FastTreeParams()
    params.set_values(*c["abg"]); params.set_q_tile_sizes(list(c["q_tiles"])); params.set_kv_tile_sizes([32, 32])
    params.set_kv_group_num(c["hq"] // c["hkv"])
    aux, _ = fasttree_preparation(tree, inp.KV_ptrs, batch, c["hq"], c["hkv"], c["d"], list(c["splits"]),
                                  list(c["thr"][0]), list(c["thr"][1]), params, device=device, kv_slot_map=inp.slot_map,
                                  launch_order=c["launch_order"])
    scale = 1.0 / math.sqrt(c["d"])
    o = torch.full_like(inp.Q, float("nan"))
    fasttree_decode(inp.Q, inp.K_pool, inp.V_pool, o, *aux, list(params.TSQs), list(params.TSKs), scale)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()
    # every request against the decode over gathered caches (another plan, another kernel path)
    k_cache, v_cache, seqlens = gather_per_request(inp)
    o_g = torch.empty_like(o)
    gathered_decode(inp.Q, k_cache, v_cache, seqlens, o_g, scale)
    torch.cuda.synchronize()
    tol = 2e-3 if c["dtype"] == torch.float16 else 2e-2  # two bf16 roundings of values up to ~4
    worst = (o.float() - o_g.float()).abs().max().item()
    assert worst <= 2 * tol, f"tree vs gathered decode: {worst}"
    # sampled requests against the dense oracle, at the parity bar
    reqs = sorted(set(np.random.default_rng(seed).integers(0, batch, size=min(batch, 12)).tolist()))
    paths = [inp.path_tokens[r] for r in reqs]
    q_cpu, k_cpu, v_cpu = inp.Q.cpu(), inp.K_pool.cpu(), inp.V_pool.cpu()
    dense = oracle.dense_attention(q_cpu[reqs], k_cpu, v_cpu, paths, scale)
    if c["dtype"] == torch.bfloat16:
        p_round = oracle.dense_attention(q_cpu[reqs], k_cpu, v_cpu.abs(), paths, scale) * 2.0 ** -9
        assert_parity(o[reqs], dense, f"random {seed}", out_dtype=torch.bfloat16, extra=p_round)
        # like for like: the reference kernels' arithmetic in bfloat16 on the same plan (fasttree.py:391)
        same_type = arith_reference(q_cpu[reqs], k_cpu, v_cpu, aux, reqs, 32, scale)
        like = assert_like_for_like(o[reqs], same_type, f"random {seed}, like for like")
        raw = (o[reqs].cpu().double() - dense).abs()
        print(f"  bf16 random {seed}: vs bf16 arithmetic max-abs {like[0]:.2e} mean-abs {like[1]:.2e}; vs fp64 raw max-abs "
              f"{float(raw.max()):.2e}", flush=True)
    else:
        assert_parity(o[reqs], dense.to(torch.float16), f"random {seed}")
