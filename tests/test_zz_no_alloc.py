"""The decode entry point that allocates nothing (ft_decode_static): same output, bit for bit,
as the entry point it is a variant of (ft_decode_programs, through fasttree_decode), on two calls
in a row that share the library's scratch array, the second with a smaller input; inputs whose
partial results do not fit the array are refused."""

import math

import pytest
import torch

from cases import build_tree
from fasttree_hip import _lib
from fasttree_hip.decode import fasttree_decode, fasttree_decode_static
from fasttree_hip.inputs import make_decode_inputs
from fasttree_hip.planner import FastTreeParams, fasttree_preparation
import fasttree_hip.planner as planner_module

pytestmark = pytest.mark.gpu


def _problem(device, sizes, lens, hq, hkv, dtype, seed):
    planner_module.VERBOSE = False
    tree, ptrs, batch = build_tree({"kind": "regular", "sizes": sizes, "lens": lens})
    inp = make_decode_inputs(tree, hq, hkv, 128, device=device, dtype=dtype, seed=seed, shuffle_slots=True)
    g = hq // hkv
    params = FastTreeParams()
    params.set_values(0.66, 0.33, 0.1); params.set_q_tile_sizes([64 // g, 16 // g]); params.set_kv_tile_sizes([32, 32])
    params.set_kv_group_num(g)
    aux, _ = fasttree_preparation(tree, inp.KV_ptrs, batch, hq, hkv, 128, [1024, 256], [256, 1024], [256, 256], params,
                                  device=device, kv_slot_map=inp.slot_map, launch_order=True)
    return inp, aux, list(params.TSQs)


def test_static_scratch_entry_point_matches_the_allocating_one(device):
    scale = 1.0 / math.sqrt(128)
    cases = [([1, 10, 400], [4000, 400, 40], 32, 8, torch.float16),     # 2000 scratch rows (33 MB), block programs
             ([1, 6, 90], [700, 130, 40], 16, 4, torch.bfloat16)]       # smaller: part of the array keeps the first call's rows
    rows_seen = []
    for seed, (sizes, lens, hq, hkv, dtype) in enumerate(cases):
        print("\n[gpu case] static scratch", sizes, lens, hq, hkv, dtype, flush=True)
        inp, aux, q_tiles = _problem(device, sizes, lens, hq, hkv, dtype, seed)
        want = torch.empty_like(inp.Q)
        fasttree_decode(inp.Q, inp.K_pool, inp.V_pool, want, *aux, q_tiles, [32, 32], scale)
        got = torch.full_like(inp.Q, float("nan"))
        # a first call looks up the array's address and raises the kernels' LDS limits; the call that
        # is checked comes after it
        fasttree_decode_static(inp.Q, inp.K_pool, inp.V_pool, got, *aux[:9], aux[11], aux[12], scale)
        torch.cuda.synchronize()
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        # device-wide free memory, as the driver reports it: it also sees what the library itself
        # would allocate or free, which torch's own counters do not
        free_before, _ = torch.cuda.mem_get_info(device)
        allocated_before = torch.cuda.memory_allocated(device)
        fasttree_decode_static(inp.Q, inp.K_pool, inp.V_pool, got, *aux[:9], aux[11], aux[12], scale)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(device)
        assert free_after == free_before, f"device-wide free memory changed by {free_before - free_after} bytes"
        assert torch.cuda.memory_allocated(device) == allocated_before
        assert torch.equal(got, want), f"{sizes}: max diff {(got.float() - want.float()).abs().max().item():.3e}"
        assert getattr(aux[11], "num_programs", 0) > 0
        rows_seen.append(aux[3].numel())
    assert rows_seen[1] < rows_seen[0]


def test_static_scratch_refuses_what_does_not_fit(device):
    inp, aux, q_tiles = _problem(device, [1, 4], [64, 40], 32, 8, torch.float16, 3)
    o = torch.zeros_like(inp.Q)
    lib = _lib.load()
    capacity = lib.ft_static_scratch_bytes()
    assert capacity == 64 << 20
    rows = capacity // (32 * 129 * 4) + 1      # one row more than the array holds at 32 heads x 128 dims
    args = [inp.Q.data_ptr(), inp.K_pool.data_ptr(), inp.V_pool.data_ptr(), o.data_ptr(),
            inp.Q.stride(0), inp.Q.stride(1), inp.K_pool.stride(0), inp.K_pool.stride(1),
            inp.V_pool.stride(0), inp.V_pool.stride(1), o.stride(0), o.stride(1)]
    args += [t.data_ptr() for t in aux[:9]]
    tail = [_lib.int32_pair(aux[11]), _lib.int32_pair(aux[12]), None, 0, 0, None, None, None, inp.Q.shape[0], 32, 8, 128,
            1.0 / math.sqrt(128), 0, None]
    rc = lib.ft_decode_static(*args, rows, *tail)
    assert rc == -8 and b"static scratch" in lib.ft_error_string(rc)
    assert lib.ft_decode_static(*args, -1, *tail) == -6
    torch.cuda.synchronize()
    assert float(o.abs().max()) == 0.0, "a refused call launches nothing"
