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



def arith_reference(q, k_pool, v_pool, aux, sample, kv_tile, sm_scale, remap=None):
    """The reference kernels' own arithmetic in the storage type, for the requests ``sample`` on the
    very plan ``aux`` (see oracle.decode_arith_for_requests)."""
    import fasttree_oracle as oracle

    lists = [t.detach().cpu().numpy() for t in aux[:9]]
    return oracle.decode_arith_for_requests(q, k_pool, v_pool, lists, sample, kv_tile, sm_scale, remap=remap)


def assert_like_for_like(got, want, what="", strict=False):
    """``got`` against the reference arithmetic evaluated in the same 16-bit type (``want``, from
    :func:`arith_reference`): mean-abs at the plain bar; max-abs at the plain bar or, where one
    unit in the last place of the expected value is coarser than the bar (bfloat16 values of
    magnitude 0.5 and more: 2**-8 and up), at most that one unit -- the two results are then
    neighbouring representable values.  ``strict`` holds every element to the plain bar."""
    g = got.detach().cpu().to(torch.float64)
    w = want.detach().cpu().to(torch.float64)
    diff = (g - w).abs()
    worst_max = float(diff.max())
    worst_mean = float(diff.reshape(g.shape[0], -1).mean(dim=1).max())
    allowed = torch.full_like(w, MAX_ABS_TOL)
    if not strict:
        mant_bits = 7 if want.dtype == torch.bfloat16 else 10
        ulp = torch.exp2(torch.floor(torch.log2(w.abs().clamp_min(2.0 ** -126))) - mant_bits)
        allowed = torch.maximum(allowed, ulp)
    over = float((diff - allowed).max())
    assert over <= 0 and worst_mean <= MEAN_ABS_TOL, (
        f"{what}: like for like max-abs {worst_max:.3e} (over the allowance by {over:.3e}), mean-abs {worst_mean:.3e}")
    return worst_max, worst_mean
