"""Pins the CPU oracle (oracle/fasttree_oracle.py): against the fixtures the reference's own
planner and kernels produced, against closed forms and against brute force."""

import math

import numpy as np
import pytest
import torch

import fasttree_oracle as oracle
from cases import KERNEL_CASES, PLANNER_CASES, build_tree, digest, kernel_case_inputs
from fasttree_hip.inputs import request_paths
from helpers import bits16_to_tensor, kernel_golden, per_request_errors, planner_goldens, run_planner

ARRAYS = ["vnode_to_kv_entries", "vnode_to_kv_offs", "vnode_to_kv_lens", "vnode_to_q_entries", "vnode_to_q_offs",
          "vnode_to_q_lens", "req_to_vnode_entries", "req_to_vnode_offs", "req_to_vnode_lens", "node_assignments"]
DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module")
def goldens():
    return planner_goldens()


@pytest.mark.parametrize("case", PLANNER_CASES, ids=[c["name"] for c in PLANNER_CASES])
def test_plan_restatement_matches_reference_fixture(case, goldens):
    gold = goldens[case["name"]]
    tree, ptrs, batch = build_tree(case["tree"])
    res = oracle.plan_from_tree(tree, ptrs, batch, case)
    for name in ARRAYS:
        arr = np.asarray(getattr(res, name), dtype=np.int32)
        assert arr.size == gold[name]["len"] and digest(arr) == gold[name]["sha256"], name
    assert res.phase_node_nums == gold["phase_node_nums"] and res.phase_node_offsets == gold["phase_node_offsets"]
    assert res.final_TSQs == gold["final_TSQs"] and res.final_TSKs == gold["final_TSKs"]
    assert res.stdout == gold["stdout"]


def _kernel_case(case):
    tree, ptrs, batch, plan, params, _ = run_planner(case)
    q, k, v = kernel_case_inputs(case, tree, ptrs, batch)
    gold = kernel_golden(case["name"])
    # the fixture's inputs are rebuilt from the seed: make sure they are the same bits
    assert digest(q.view(torch.int16).numpy()) == str(gold["q_sha256"])
    assert digest(k.view(torch.int16).numpy()) == str(gold["k_sha256"])
    assert digest(v.view(torch.int16).numpy()) == str(gold["v_sha256"])
    return tree, ptrs, batch, plan, q, k, v, gold


@pytest.mark.parametrize("case", KERNEL_CASES, ids=[c["name"] for c in KERNEL_CASES])
def test_two_stage_arithmetic_matches_reference_kernels(case):
    """mid_o, mid_lse and o of the restated arithmetic agree with what the reference's Triton
    kernels wrote (CPU interpreter) far inside the parity tolerance: only the summation
    order inside the dot products differs."""
    tree, ptrs, batch, plan, q, k, v, gold = _kernel_case(case)
    sm_scale = 1.0 / math.sqrt(case["D"])
    o, mid_o, mid_lse = oracle.fasttree_decode_arith(q, k, v, plan, case["TSKs"][0], sm_scale)
    if "mid_o" in gold:      # (the full-size fixtures hold the outputs of a request subset only)
        assert torch.allclose(mid_lse, torch.from_numpy(gold["mid_lse"]), rtol=0, atol=2e-5)
        assert torch.allclose(mid_o, torch.from_numpy(gold["mid_o"]), rtol=0, atol=2e-4 if case["dtype"] == "fp16" else 2e-3)
    if "requests" in gold:
        o = o[gold["requests"].tolist()]
    want = bits16_to_tensor(gold["o"], DTYPES[case["dtype"]])
    worst_max, worst_mean = per_request_errors(o, want)
    one_ulp = 2e-3 if case["dtype"] == "fp16" else 1.6e-2      # outputs are O(1): half / bfloat16 spacing near 2
    assert worst_max <= one_ulp and worst_mean <= one_ulp / 20


@pytest.mark.parametrize("case", KERNEL_CASES, ids=[c["name"] for c in KERNEL_CASES])
def test_arithmetic_for_sampled_requests_matches_reference_kernels(case):
    """decode_arith_for_requests (the two-stage arithmetic for a few requests of a plan, what the
    bfloat16 GPU cases are compared with like for like) against what the reference's own kernels
    wrote for those requests, and against fasttree_decode_arith on the whole plan: restricting a
    plan to some of its requests changes nothing for them."""
    tree, ptrs, batch, plan, q, k, v, gold = _kernel_case(case)
    sm_scale = 1.0 / math.sqrt(case["D"])
    kept = gold["requests"].tolist() if "requests" in gold else list(range(batch))
    want = bits16_to_tensor(gold["o"], DTYPES[case["dtype"]])
    picks = sorted(set(range(0, len(kept), max(1, len(kept) // 5))))        # positions within the fixture's requests
    sample = [kept[i] for i in picks]
    lists = [np.asarray(getattr(plan, name)) for name in ARRAYS[:9]]
    o = oracle.decode_arith_for_requests(q[sample], k, v, lists, sample, case["TSKs"][0], sm_scale)
    worst_max, worst_mean = per_request_errors(o, want[picks])
    one_ulp = 2e-3 if case["dtype"] == "fp16" else 1.6e-2
    assert worst_max <= one_ulp and worst_mean <= one_ulp / 20
    full, _, _ = oracle.fasttree_decode_arith(q, k, v, plan, case["TSKs"][0], sm_scale)
    assert torch.allclose(o.float(), full[sample].float(), rtol=0, atol=1e-3 if case["dtype"] == "fp16" else 8e-3)
    assert (o.float() - full[sample].float()).abs().mean() <= 2e-5


@pytest.mark.parametrize("case", KERNEL_CASES, ids=[c["name"] for c in KERNEL_CASES])
def test_dense_identity_matches_reference_kernels(case):
    """Tree attention == dense soft-max attention of each request over its root path."""
    tree, ptrs, batch, plan, q, k, v, gold = _kernel_case(case)
    want = bits16_to_tensor(gold["o"], DTYPES[case["dtype"]])
    paths = request_paths(tree, ptrs)
    if "requests" in gold:   # a full-size case: the fixture holds a request subset
        kept = gold["requests"].tolist()
        q, paths = q[kept], [paths[r] for r in kept]
    dense = oracle.dense_attention(q, k, v, paths, 1.0 / math.sqrt(case["D"]))
    worst_max, worst_mean = per_request_errors(dense, want)
    if case["dtype"] == "fp16":
        assert worst_max <= 2e-3 and worst_mean <= 1e-3
    else:  # bfloat16 outputs carry 8 bits: one ulp near 1 is 7.8e-3
        assert worst_max <= 1.6e-2 and worst_mean <= 2e-3
    fast = oracle.gathered_attention_torch(q, k, v, paths, 1.0 / math.sqrt(case["D"]))
    assert torch.allclose(fast.double(), dense, atol=2e-5, rtol=0)


def test_dense_closed_forms():
    d = 16
    q = torch.randn(2, 4, d, dtype=torch.float64)
    k = torch.randn(5, 2, d, dtype=torch.float64)
    v = torch.randn(5, 2, d, dtype=torch.float64)
    # one key: the output is that key's value whatever the score
    out = oracle.dense_attention(q, k, v, [np.array([3]), np.array([1])], 0.7)
    assert torch.allclose(out[0, :2], v[3, 0].expand(2, d)) and torch.allclose(out[1, 2:], v[1, 1].expand(2, d))
    # identical keys: uniform weights, the output is the mean of the values
    k_same = k[:1].expand(5, 2, d).contiguous()
    out = oracle.dense_attention(q, k_same, v, [np.arange(5), np.arange(5)], 0.7)
    assert torch.allclose(out[0, 0], v[:, 0].mean(dim=0)) and torch.allclose(out[1, 3], v[:, 1].mean(dim=0))
    # brute force with python loops, GQA head mapping h -> h // g
    path = np.array([4, 0, 2])
    out = oracle.dense_attention(q, k, v, [path, path], 0.3)
    for r in range(2):
        for h in range(4):
            w = [math.exp(0.3 * float(q[r, h] @ k[t, h // 2])) for t in path]
            want = sum(wi * v[t, h // 2] for wi, t in zip(w, path)) / sum(w)
            assert torch.allclose(out[r, h], want)


def test_stage_split_invariance_and_lse_semantics():
    """Any cut of the KV run gives the same merged result; mid_lse is the natural-log
    log-sum-exp of the scaled scores and mid_o the partial normalised by its own sum."""
    torch.manual_seed(0)
    d, hq, hkv, total = 32, 4, 2, 77
    q = torch.randn(1, hq, d).half()
    k = torch.randn(total, hkv, d).half()
    v = torch.randn(total, hkv, d).half()
    scale = 1 / math.sqrt(d)
    dense = oracle.dense_attention(q, k, v, [np.arange(total)], scale)
    for cuts in ([0, 77], [0, 10, 77], [0, 32, 64, 77], [0, 1, 2, 76, 77]):
        offs, lens = cuts[:-1], [b - a for a, b in zip(cuts[:-1], cuts[1:])]
        rows = len(offs)
        mid_o, mid_lse = oracle.stage1_arith(q, k, v, np.arange(total), offs, lens, [0] * rows, list(range(rows)),
                                             [1] * rows, 32, scale, rows)
        o = oracle.stage2_arith(list(range(rows)), [0], [rows], mid_o, mid_lse, torch.float32)
        assert torch.allclose(o.double(), dense, atol=2e-3)
        for i, (a, n) in enumerate(zip(offs, lens)):
            s = torch.einsum("hd,thd->ht", q[0].double(), k[a:a + n].double().repeat_interleave(2, dim=1)) * scale
            assert torch.allclose(mid_lse[i].double(), torch.logsumexp(s, dim=-1), atol=1e-5)
            part = oracle.dense_attention(q, k, v, [np.arange(a, a + n)], scale)
            assert torch.allclose(mid_o[i].double(), part[0], atol=2e-3)


def test_stage2_single_partial_and_order():
    mid_o = torch.randn(3, 2, 8)
    mid_lse = torch.randn(3, 2)
    one = oracle.stage2_arith([1], [0], [1], mid_o, mid_lse, torch.float32)
    assert torch.allclose(one[0], mid_o[1])
    a = oracle.stage2_arith([0, 1, 2], [0], [3], mid_o, mid_lse, torch.float32)
    b = oracle.stage2_arith([2, 0, 1], [0], [3], mid_o, mid_lse, torch.float32)
    w = torch.softmax(mid_lse, dim=0)
    assert torch.allclose(a, b, atol=1e-6) and torch.allclose(a[0], (w[..., None] * mid_o).sum(dim=0), atol=1e-6)
