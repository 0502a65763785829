#!/usr/bin/env python3
"""Writes the golden fixtures in this directory by running the reference's own planner
and (under Triton's CPU interpreter) its own two decode kernels.

Run once in a container that holds the reference checkout; the fixtures it writes are
plain data (JSON / npz) and are what the tests read -- nothing in the test suite, the
smoke run or the bench imports the reference.

    python tests/golden/make_goldens.py [--reference /root/reference] [--only planner|kernel|deft]

What is taken from the reference: ``_tree_heuristic``, ``fasttree_preparation``,
``FastTreeParams`` and ``fasttree_decode`` of kernel_bench/fasttree.py.  Because that
planner hard-wires ``torch.device("cuda")`` for its output tensors
(kernel_bench/fasttree.py:265), the module's ``torch`` name is pointed at a thin proxy
whose ``device()`` is a no-op context so the tensors land on the CPU; nothing else is
altered.  Inputs (trees, requests, Q/K/V) are built by this repository's own generators.

``--only deft`` writes ``deft_*.npz``: the index arrays and masks of the reference's
``DeFT_preparation`` and the outputs of its ``DeFT_decode`` (kernel_bench/DeFT.py, the comparison
engine of the reference's benchmark) under the same interpreter, on the per-request gathered
cache that engine reads.
"""

from __future__ import annotations

import argparse
import contextlib
import hashlib
import importlib.util
import io
import json
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "fasttree-artifact_amd"))
sys.path.insert(0, HERE)

import numpy as np  # noqa: E402

from cases import (  # noqa: E402
    KERNEL_CASES, PLANNER_CASES, build_tree, make_params_kwargs, kernel_case_inputs, digest,
)

FULL_ARRAY_LIMIT = 256  # longer integer arrays are stored as sha256 + head/tail


def load_reference(ref_root: str):
    os.environ["TRITON_INTERPRET"] = "1"
    import torch

    path = os.path.join(ref_root, "kernel_bench", "fasttree.py")
    spec = importlib.util.spec_from_file_location("_reference_fasttree", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)

    class _HostTorch:
        def __getattr__(self, name):
            return getattr(torch, name)

        @staticmethod
        def device(*_a, **_k):
            return contextlib.nullcontext()

    mod.torch = _HostTorch()
    return mod


def pack_ints(values) -> dict:
    arr = np.asarray(values, dtype=np.int32).reshape(-1)
    rec = {"len": int(arr.size), "sha256": digest(arr)}
    if arr.size <= FULL_ARRAY_LIMIT:
        rec["values"] = arr.tolist()
    else:
        rec["head"] = arr[:64].tolist()
        rec["tail"] = arr[-64:].tolist()
    return rec


def reference_params(ref, kw):
    p = ref.FastTreeParams()
    p.set_values(kw["alpha"], kw["beta"], kw["gamma"])
    p.set_q_tile_sizes(list(kw["TSQs"]))
    p.set_kv_tile_sizes(list(kw["TSKs"]))
    p.set_kv_group_num(kw["kv_group_num"])
    return p


def run_reference_planner(ref, case):
    tree, ptrs, batch = build_tree(case["tree"])
    kw = make_params_kwargs(case)
    params = reference_params(ref, kw)
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        aux, assignment = ref.fasttree_preparation(
            tree, ptrs, batch, case["Hq"], case["Hkv"], case["D"],
            list(case["kv_split_sizes"]), list(case["para_threshs1"]), list(case["para_threshs2"]), params,
        )
    return tree, ptrs, batch, aux, assignment, params, out.getvalue()


def planner_goldens(ref) -> dict:
    records = {}
    for case in PLANNER_CASES:
        t0 = time.time()
        _, _, batch, aux, assignment, params, text = run_reference_planner(ref, case)
        names = [
            "vnode_to_kv_entries", "vnode_to_kv_offs", "vnode_to_kv_lens",
            "vnode_to_q_entries", "vnode_to_q_offs", "vnode_to_q_lens",
            "req_to_vnode_entries", "req_to_vnode_offs", "req_to_vnode_lens",
        ]
        rec = {"case": case, "batch_size": batch}
        for name, tensor in zip(names, aux[:9]):
            rec[name] = pack_ints(tensor.numpy())
        rec["mid_o_shape"] = list(aux[9].shape)
        rec["mid_lse_shape"] = list(aux[10].shape)
        rec["phase_node_nums"] = [int(x) for x in aux[11]]
        rec["phase_node_offsets"] = [int(x) for x in aux[12]]
        rec["node_assignments"] = pack_ints(assignment)
        rec["final_TSQs"] = [int(x) for x in params.TSQs]
        rec["final_TSKs"] = [int(x) for x in params.TSKs]
        rec["stdout"] = text
        records[case["name"]] = rec
        print(f"planner {case['name']}: {time.time() - t0:.1f}s", file=sys.stderr)
    return records


def kernel_goldens(ref, out_dir: str, names=None):
    import torch

    for case in KERNEL_CASES:
        if names and case["name"] not in names:
            continue
        t0 = time.time()
        tree, ptrs, batch, aux, assignment, params, _ = run_reference_planner(ref, case)
        q, k_pool, v_pool = kernel_case_inputs(case, tree, ptrs, batch)
        o = torch.zeros_like(q)
        # The bench passes its own tile lists, not the planner's final ones
        # (kernel_bench/benchmark.py:121-122); the cases here are chosen so both agree.
        assert list(params.TSQs) == list(case["TSQs"]), case["name"]
        sm_scale = 1.0 / (case["D"] ** 0.5)
        ref.fasttree_decode(q, k_pool, v_pool, o, *aux, list(case["TSQs"]), list(case["TSKs"]), sm_scale)
        rows = aux[3].numel()
        if case.get("keep_every"):
            # a full-size case: the outputs of a request subset only (the partial results of
            # such a launch run to tens of megabytes)
            kept = np.arange(0, batch, case["keep_every"])
            np.savez_compressed(
                os.path.join(out_dir, f"kernel_{case['name']}.npz"),
                o=o[torch.from_numpy(kept)].view(torch.int16).numpy(), requests=kept,
                q_sha256=np.array(digest(q.view(torch.int16).numpy())),
                k_sha256=np.array(digest(k_pool.view(torch.int16).numpy())),
                v_sha256=np.array(digest(v_pool.view(torch.int16).numpy())),
            )
            print(f"kernel {case['name']}: {time.time() - t0:.1f}s", file=sys.stderr)
            continue
        np.savez_compressed(
            os.path.join(out_dir, f"kernel_{case['name']}.npz"),
            o=o.view(torch.int16).numpy(),                       # raw 16-bit patterns
            mid_o=aux[9][:rows].numpy(),
            mid_lse=aux[10][:rows].numpy(),
            q_sha256=np.array(digest(q.view(torch.int16).numpy())),
            k_sha256=np.array(digest(k_pool.view(torch.int16).numpy())),
            v_sha256=np.array(digest(v_pool.view(torch.int16).numpy())),
        )
        print(f"kernel {case['name']}: {time.time() - t0:.1f}s", file=sys.stderr)


def load_reference_deft(ref_root: str):
    os.environ["TRITON_INTERPRET"] = "1"
    import torch

    bench_dir = os.path.join(ref_root, "kernel_bench")
    sys.path.insert(0, bench_dir)            # DeFT.py imports kv_tree_simple from its own directory
    try:
        spec = importlib.util.spec_from_file_location("_reference_deft", os.path.join(bench_dir, "DeFT.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
    finally:
        sys.path.remove(bench_dir)

    class _HostTorch:
        def __getattr__(self, name):
            return getattr(torch, name)

        @staticmethod
        def device(*_a, **_k):
            return contextlib.nullcontext()

    mod.torch = _HostTorch()
    return mod


def deft_goldens(ref_root: str, out_dir: str):
    import torch

    from cases import DEFT_CASES, gathered_cache

    ref = load_reference_deft(ref_root)
    names = ["vnode_to_kv_entries", "vnode_to_kv_offs", "vnode_to_kv_lens", "vnode_to_q_entries", "vnode_to_q_offs",
             "vnode_to_q_lens", "causalmask", "causalmask_offset", "req_to_vnode_entries", "req_to_vnode_offs",
             "req_to_vnode_lens"]
    for case in DEFT_CASES:
        t0 = time.time()
        tree, ptrs, batch = build_tree(case["tree"])
        q, k_pool, v_pool = kernel_case_inputs(case, tree, ptrs, batch)
        k_cache, v_cache = gathered_cache(tree, ptrs, k_pool, v_pool)
        ref.cur_length = 0                   # (a module global the partition accumulates in, DeFT.py:26)
        aux = ref.DeFT_preparation(tree, k_cache, case["subtree_len"], case["mask_len"], case["Hq"], case["D"])
        o = torch.zeros_like(q)
        sm_scale = 1.0 / (case["D"] ** 0.5)
        ref.DeFT_decode(q, k_cache.view(-1, case["Hkv"], case["D"]), v_cache.view(-1, case["Hkv"], case["D"]), o, *aux,
                        case["q_tile"], 32, sm_scale, case["mask_len"])
        record = {name: t.numpy() for name, t in zip(names, aux[:11])}
        np.savez_compressed(
            os.path.join(out_dir, f"deft_{case['name']}.npz"),
            o=o.view(torch.int16).numpy(), mid_o=aux[11].numpy(), mid_lse=aux[12].numpy(),
            q_sha256=np.array(digest(q.view(torch.int16).numpy())),
            k_sha256=np.array(digest(k_cache.view(torch.int16).numpy())),
            v_sha256=np.array(digest(v_cache.view(torch.int16).numpy())),
            **record,
        )
        print(f"deft {case['name']}: {time.time() - t0:.1f}s, {len(aux[1])} subtrees", file=sys.stderr)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reference", default="/root/reference")
    ap.add_argument("--only", choices=["planner", "kernel", "deft"], default=None)
    ap.add_argument("--cases", default=None, help="kernel cases to (re)write, comma separated (default: all)")
    args = ap.parse_args()
    if args.only in (None, "deft"):
        deft_goldens(args.reference, HERE)
        if args.only == "deft":
            return
    ref = load_reference(args.reference)
    if args.only in (None, "planner"):
        with open(os.path.join(HERE, "planner_goldens.json"), "w") as fh:
            json.dump(planner_goldens(ref), fh, separators=(",", ":"))
    if args.only in (None, "kernel"):
        kernel_goldens(ref, HERE, args.cases.split(",") if args.cases else None)


if __name__ == "__main__":
    main()
