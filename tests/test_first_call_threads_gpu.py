"""Two host threads make their first decode call at the same time, in a fresh process: the
library's per-device set-up (raising the kernels' LDS limits, reading the device's size) is done by
whichever thread comes first, or by both, and both calls give the right result."""

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r'''
import math, sys, threading
sys.path[:0] = [{pkg!r}, {golden!r}, {oracle!r}]
import torch
import fasttree_oracle as oracle
from cases import build_tree
import fasttree_hip.planner as planner_module
from fasttree_hip.decode import fasttree_decode
from fasttree_hip.inputs import make_decode_inputs
from fasttree_hip.planner import FastTreeParams, fasttree_preparation

planner_module.VERBOSE = False
device = torch.device("cuda:0")
torch.cuda.set_device(device)
scale = 1.0 / math.sqrt(128)

def problem(seed, launch_order):
    tree, ptrs, batch = build_tree({{"kind": "regular", "sizes": [1, 4, 40], "lens": [500, 100, 30]}})
    inp = make_decode_inputs(tree, 32, 8, 128, device=device, dtype=torch.float16, seed=seed, shuffle_slots=True)
    params = FastTreeParams()
    params.set_values(0.66, 0.33, 0.1); params.set_q_tile_sizes([16, 4]); params.set_kv_tile_sizes([32, 32])
    params.set_kv_group_num(4)
    aux, _ = fasttree_preparation(tree, inp.KV_ptrs, batch, 32, 8, 128, [1024, 256], [256, 1024], [256, 256], params,
                                  device=device, kv_slot_map=inp.slot_map, launch_order=launch_order)
    return inp, aux, list(params.TSQs)

# everything but the library's first call happens before the threads start
work = [problem(0, True), problem(1, False)]
outs = [torch.full_like(w[0].Q, float("nan")) for w in work]
streams = [torch.cuda.Stream(device) for _ in work]
torch.cuda.synchronize()
gate = threading.Barrier(2)
errors = []

def call(i):
    try:
        inp, aux, q_tiles = work[i]
        with torch.cuda.stream(streams[i]):
            gate.wait()
            fasttree_decode(inp.Q, inp.K_pool, inp.V_pool, outs[i], *aux, q_tiles, [32, 32], scale)
        streams[i].synchronize()
    except Exception as exc:      # reported by the parent
        errors.append(repr(exc))

threads = [threading.Thread(target=call, args=(i,)) for i in range(2)]
for t in threads: t.start()
for t in threads: t.join()
assert not errors, errors
for (inp, aux, _), o in zip(work, outs):
    want = oracle.dense_attention(inp.Q.cpu(), inp.K_pool.cpu(), inp.V_pool.cpu(), inp.path_tokens, scale)
    diff = (o.cpu().double() - want).abs().reshape(o.shape[0], -1)
    assert float(diff.max()) <= 2e-3 and float(diff.mean(dim=1).max()) <= 1e-3, float(diff.max())
print("threads ok")
'''


def test_two_threads_make_the_first_call_together(device):
    print("\n[gpu case] first decode call from two threads at once (child process)", flush=True)
    code = CHILD.format(pkg=os.path.join(ROOT, "fasttree-artifact_amd"), golden=os.path.join(ROOT, "tests", "golden"),
                        oracle=os.path.join(ROOT, "oracle"))
    done = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and "threads ok" in done.stdout, done.stdout[-2000:] + done.stderr[-4000:]
