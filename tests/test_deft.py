"""DeFT-Flatten, the comparison engine of the reference's benchmark (kernel_bench/DeFT.py), as
built here: the preparation's index arrays and masks bit for bit against what the reference's own
``DeFT_preparation`` wrote (tests/golden/deft_*.npz, written by tests/golden/make_goldens.py), and
-- on the GPU -- ``DeFT_decode`` against the outputs of the reference's own Triton kernels (run
under Triton's CPU interpreter for those fixtures) and against the fp64 dense oracle."""
import math
import os
import sys

import numpy as np
import pytest
import torch

import fasttree_oracle as oracle
from cases import DEFT_CASES, build_tree, digest, gathered_cache, kernel_case_inputs
from fasttree_hip.inputs import request_paths
from helpers import GOLDEN_DIR, assert_parity, bits16_to_tensor

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fasttree-artifact_amd", "kernel_bench"))
import DeFT  # noqa: E402

NAMES = ["vnode_to_kv_entries", "vnode_to_kv_offs", "vnode_to_kv_lens", "vnode_to_q_entries", "vnode_to_q_offs",
         "vnode_to_q_lens", "causalmask", "causalmask_offset", "req_to_vnode_entries", "req_to_vnode_offs",
         "req_to_vnode_lens"]


def _golden(case):
    return np.load(os.path.join(GOLDEN_DIR, f"deft_{case['name']}.npz"))


def _inputs(case):
    tree, ptrs, batch = build_tree(case["tree"])
    q, k_pool, v_pool = kernel_case_inputs(case, tree, ptrs, batch)
    k_cache, v_cache = gathered_cache(tree, ptrs, k_pool, v_pool)
    return tree, ptrs, batch, q, k_pool, v_pool, k_cache, v_cache


@pytest.mark.parametrize("case", DEFT_CASES, ids=[c["name"] for c in DEFT_CASES])
def test_preparation_matches_the_reference_arrays(case):
    tree, ptrs, batch, q, k_pool, v_pool, k_cache, v_cache = _inputs(case)
    gold = _golden(case)
    got = DeFT.deft_lists(tree, batch, k_cache.shape[1], case["subtree_len"], case["mask_len"])
    for name, arr in zip(NAMES, got):
        want = gold[name]
        assert arr.dtype == want.dtype and arr.shape == want.shape and np.array_equal(arr, want), name
    aux = DeFT.DeFT_preparation(tree, k_cache, case["subtree_len"], case["mask_len"], case["Hq"], case["D"], device="cpu")
    assert len(aux) == 13 and aux[6].dtype == torch.int64 and all(t.dtype == torch.int32 for i, t in enumerate(aux[:11]) if i != 6)
    assert tuple(aux[11].shape) == (len(gold["vnode_to_q_entries"]), case["Hq"], case["D"]) == tuple(gold["mid_o"].shape)
    assert tuple(aux[12].shape) == tuple(gold["mid_lse"].shape) and aux[11].dtype == aux[12].dtype == torch.float32


def test_partition_hand_case():
    """kat1 tree (nodes of 100, 50, 10, 10 tokens; requests 0 and 1) in subtrees of 32 tokens, by
    hand from DeFT.py:29-55: the root fills three subtrees and opens the fourth with 4 tokens,
    node 1 adds 28, fills the fifth and opens the sixth with its last 22, which the two leaves
    complete -- depth first, node 2 before node 3."""
    tree, ptrs, batch = build_tree(DEFT_CASES[0]["tree"])
    assert DeFT.group_subtree(tree, 32) == [
        [(0, 0, 32)], [(0, 32, 64)], [(0, 64, 96)], [(0, 96, 100), (1, 0, 28)], [(1, 28, 50), (2, 0, 10)], [(3, 0, 10)]]
    lists = DeFT.deft_lists(tree, batch, 160, 32, 64)
    # both requests attend the root and node 1, request 0 alone node 2, request 1 alone node 3
    assert lists[3].tolist() == [0, 1] * 5 + [1] and lists[5].tolist() == [2, 2, 2, 2, 2, 1]
    assert lists[6].tolist() == [3] * 32 * 4 + [3] * 22 + [1] * 10 + [1] * 10
    assert lists[8].tolist()[:-32] == [0, 2, 4, 6, 8, 1, 3, 5, 7, 9, 10] and lists[10].tolist() == [5, 6]
    # a node without tokens still brings its requests into the query set of the subtree it falls in
    tree[2].seqlen = 0
    assert DeFT.group_subtree(tree, 32)[4] == [(1, 28, 50), (2, 0, 0), (3, 0, 10)]


@pytest.mark.parametrize("case", DEFT_CASES, ids=[c["name"] for c in DEFT_CASES])
def test_reference_outputs_satisfy_the_dense_identity(case):
    """What the reference's DeFT kernels wrote is dense soft-max attention of every request over
    its root path (the identity the GPU test below leans on for larger inputs)."""
    tree, ptrs, batch, q, k_pool, v_pool, k_cache, v_cache = _inputs(case)
    gold = _golden(case)
    assert digest(q.view(torch.int16).numpy()) == str(gold["q_sha256"])
    assert digest(k_cache.view(torch.int16).numpy()) == str(gold["k_sha256"])
    dense = oracle.dense_attention(q, k_pool, v_pool, request_paths(tree, ptrs), 1.0 / math.sqrt(case["D"]))
    assert_parity(bits16_to_tensor(gold["o"], torch.float16), dense.to(torch.float16), case["name"])


@pytest.mark.gpu
@pytest.mark.parametrize("case", DEFT_CASES, ids=[c["name"] for c in DEFT_CASES])
def test_decode_matches_the_reference_kernels(case, device):
    print("\n[gpu case] DeFT", case["name"], flush=True)
    tree, ptrs, batch, q, k_pool, v_pool, k_cache, v_cache = _inputs(case)
    gold = _golden(case)
    aux = DeFT.DeFT_preparation(tree, k_cache, case["subtree_len"], case["mask_len"], case["Hq"], case["D"], device=device)
    qd, kd, vd = q.to(device), k_cache.to(device), v_cache.to(device)
    o = torch.full_like(qd, float("nan"))
    aux[11].fill_(float("nan")); aux[12].fill_(float("nan"))
    DeFT.DeFT_decode(qd, kd.view(-1, case["Hkv"], case["D"]), vd.view(-1, case["Hkv"], case["D"]), o, *aux,
                     case["q_tile"], 32, 1.0 / math.sqrt(case["D"]), case["mask_len"])
    torch.cuda.synchronize()
    assert_parity(o, bits16_to_tensor(gold["o"], torch.float16), case["name"])
    assert_parity(aux[11], torch.from_numpy(gold["mid_o"]), case["name"] + " mid_o")
    lse_err = (aux[12].cpu() - torch.from_numpy(gold["mid_lse"])).abs().max()
    assert lse_err <= 1e-3, f"mid_lse {lse_err}"
    dense = oracle.dense_attention(q, k_pool, v_pool, request_paths(tree, ptrs), 1.0 / math.sqrt(case["D"]))
    assert_parity(o, dense.to(torch.float16), case["name"] + " vs dense")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape", [([1, 10, 400], [4000, 400, 40], 32, 8, 128), ([1, 16], [1024, 128], 32, 32, 128),
                                   ([1, 4, 40], [300, 260, 33], 16, 2, 256), ([1, 5, 150], [129, 64, 3], 8, 8, 64)],
                         ids=["c3", "c1", "d256_gqa8", "d64_mha"])
def test_decode_on_the_tree_pool_against_the_dense_oracle(shape, dtype, device):
    """Larger trees (the headline tree among them), entries addressing the shuffled tree pool
    instead of a gathered cache, fp16 and bf16: sampled requests against the fp64 oracle."""
    from fasttree_hip.inputs import make_decode_inputs
    sizes, lens, hq, hkv, d = shape
    print("\n[gpu case] DeFT on the pool", shape, dtype, flush=True)
    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": sizes, "lens": lens})
    inp = make_decode_inputs(tree, hq, hkv, d, device=device, dtype=dtype, seed=5, shuffle_slots=True)
    width = max(len(p) for p in inp.path_tokens)
    shape_only = torch.empty((batch, width, 0))
    aux = DeFT.DeFT_preparation(tree, shape_only, 128, 64, hq, d, device=device, KV_ptrs=inp.KV_ptrs, kv_slot_map=inp.slot_map)
    o = torch.full_like(inp.Q, float("nan"))
    scale = 1.0 / math.sqrt(d)
    DeFT.DeFT_decode(inp.Q, inp.K_pool, inp.V_pool, o, *aux, 16, 32, scale, 64)
    torch.cuda.synchronize()
    sample = list(range(0, batch, max(1, batch // 24)))
    dense = oracle.dense_attention(inp.Q[sample].cpu(), inp.K_pool.cpu(), inp.V_pool.cpu(), [inp.path_tokens[r] for r in sample], scale)
    if dtype == torch.bfloat16:
        assert_parity(o[sample], dense, f"DeFT {shape} bf16", out_dtype=torch.bfloat16)
    else:
        assert_parity(o[sample], dense.to(dtype), f"DeFT {shape}")
