"""Shared helpers of the test suite (not collected by pytest)."""

from __future__ import annotations

import contextlib
import io
import json
import os

import numpy as np
import torch

from cases import build_tree, make_params_kwargs
from fasttree_hip.planner import FastTreeParams, fasttree_plan

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# Parity bar of the decode path: per request, against the reference kernel's output (or the
# fp64 dense oracle where no reference output exists).
MAX_ABS_TOL = 2e-3
MEAN_ABS_TOL = 1e-3


def planner_goldens():
    with open(os.path.join(GOLDEN_DIR, "planner_goldens.json")) as fh:
        return json.load(fh)


def kernel_golden(name):
    return np.load(os.path.join(GOLDEN_DIR, f"kernel_{name}.npz"))


def params_for(case) -> FastTreeParams:
    kw = make_params_kwargs(case)
    p = FastTreeParams()
    p.set_values(kw["alpha"], kw["beta"], kw["gamma"])
    p.set_q_tile_sizes(list(kw["TSQs"]))
    p.set_kv_tile_sizes(list(kw["TSKs"]))
    p.set_kv_group_num(kw["kv_group_num"])
    return p


def run_planner(case, kv_slot_map=None, backend=None):
    """Product planner on a golden case: (tree, ptrs, batch, plan, params, stdout)."""
    tree, ptrs, batch = build_tree(case["tree"])
    params = params_for(case)
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        plan = fasttree_plan(tree, ptrs, batch, case["Hkv"], case["kv_split_sizes"], case["para_threshs1"],
                             case["para_threshs2"], params, kv_slot_map=kv_slot_map, backend=backend)
    return tree, ptrs, batch, plan, params, out.getvalue()


def bits16_to_tensor(arr: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(arr)).view(dtype)


def per_request_errors(got: torch.Tensor, want: torch.Tensor):
    """(max over requests of max-abs, max over requests of mean-abs), computed in fp64."""
    diff = (got.detach().cpu().to(torch.float64) - want.detach().cpu().to(torch.float64)).abs()
    flat = diff.reshape(diff.shape[0], -1)
    return float(flat.max(dim=1).values.max()), float(flat.mean(dim=1).max())


def assert_parity(got, want, what="", out_dtype=None, extra=None):
    """Per-request parity bar.  For bfloat16 outputs the storage grid (8 significant bits,
    spacing up to 7.8e-3 near 1) is coarser than the bar itself, so ``want`` is given
    unrounded and every element is allowed, on top of the bar, the half-ulp rounding error
    that writing it as bfloat16 incurs (at most |want| * 2**-8) plus ``extra`` (elementwise,
    optional: a bound on an error source inherent to the algorithm in that type)."""
    if out_dtype == torch.bfloat16:
        g = got.detach().cpu().to(torch.float64)
        w = want.detach().cpu().to(torch.float64)
        allowed = w.abs() * 2.0 ** -8
        if extra is not None:
            allowed = allowed + extra.detach().cpu().to(torch.float64)
        excess = ((g - w).abs() - allowed).clamp_min(0).reshape(g.shape[0], -1)
        worst_max = float(excess.max())
        worst_mean = float((g - w).abs().reshape(g.shape[0], -1).mean(dim=1).max())
    else:
        worst_max, worst_mean = per_request_errors(got, want)
    assert worst_max <= MAX_ABS_TOL and worst_mean <= MEAN_ABS_TOL, (
        f"{what}: max-abs {worst_max:.3e} (tol {MAX_ABS_TOL}), mean-abs {worst_mean:.3e} (tol {MEAN_ABS_TOL})")
    return worst_max, worst_mean


def plan_to_device(plan, hq, d, device):
    """Upload a host plan: the 13-tuple ``fasttree_preparation`` returns."""
    def put(x):
        return torch.from_numpy(np.ascontiguousarray(np.asarray(x, dtype=np.int32))).to(device)

    rows = len(plan.vnode_to_q_entries)
    return (
        put(plan.vnode_to_kv_entries), put(plan.vnode_to_kv_offs), put(plan.vnode_to_kv_lens),
        put(plan.vnode_to_q_entries), put(plan.vnode_to_q_offs), put(plan.vnode_to_q_lens),
        put(plan.req_to_vnode_entries), put(plan.req_to_vnode_offs), put(plan.req_to_vnode_lens),
        torch.full((rows, hq, d), float("nan"), dtype=torch.float32, device=device),
        torch.full((rows, hq), float("nan"), dtype=torch.float32, device=device),
        list(plan.phase_node_nums), list(plan.phase_node_offsets),
    )
