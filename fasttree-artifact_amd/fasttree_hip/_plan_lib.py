"""ctypes binding of libfasttree_plan.so, the native host planner (include/fasttree_plan.h)."""

from __future__ import annotations

import ctypes
import os

import numpy as np

LIB_NAME = "libfasttree_plan.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

# order of the result arrays (enum in include/fasttree_plan.h)
(KV_ENTRIES, KV_OFFS, KV_LENS, Q_ENTRIES, Q_OFFS, Q_LENS, REQ_ENTRIES, REQ_OFFS, REQ_LENS, NODE_ASSIGNMENTS,
 PARALLELISMS, PHASE_NODE_NUMS, PHASE_NODE_OFFSETS, Q_TILE_SIZES, KV_SPLIT_SIZES, KV_TILE_SIZES, TILES_REPLACED,
 N_ARRAYS) = range(18)

_ERRORS = {-1: "null pointer", -2: "invalid argument", -3: "out of memory"}

_P32 = ctypes.POINTER(ctypes.c_int32)
_P64 = ctypes.POINTER(ctypes.c_int64)
SIGNATURES = {
    "ft_plan_version": (ctypes.c_char_p, []),
    "ft_plan_create": (ctypes.c_int, [ctypes.c_int, _P32, _P32, _P32, _P64, _P32, _P64, ctypes.c_int, ctypes.c_int,
                                      _P32, _P32, _P32, ctypes.c_double, ctypes.c_double, ctypes.c_double, _P32, _P32,
                                      ctypes.c_int, _P32, ctypes.c_int64, ctypes.POINTER(ctypes.c_void_p)]),
    "ft_plan_size": (ctypes.c_int64, [ctypes.c_void_p, ctypes.c_int]),
    "ft_plan_copy": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, _P32, ctypes.c_int64]),
    "ft_plan_destroy": (None, [ctypes.c_void_p]),
}

_lib = None


class FastTreePlannerError(RuntimeError):
    pass


def available() -> bool:
    return os.path.exists(LIB_PATH)


def load():
    global _lib
    if _lib is None:
        if not available():
            raise FastTreePlannerError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib


def _i32(values):
    return np.ascontiguousarray(np.asarray(values, dtype=np.int32))


def _ptr32(a):
    return a.ctypes.data_as(_P32)


def plan(tree_info, KV_ptrs, batch_size, num_kv_heads, KV_SPLIT_SIZES, para_threshs1, para_threshs2,
         alpha, beta, gamma, TSQs, TSKs, kv_group_num, kv_slot_map=None):
    """Runs the native planner; returns the list of result arrays (numpy int32), indexed by the
    constants above."""
    lib = load()
    n = len(tree_info)
    parent = _i32([t.parent for t in tree_info])
    seqlen = _i32([t.seqlen for t in tree_info])
    children = _i32([t.num_children for t in tree_info])
    counts = np.fromiter((len(t.requests) for t in tree_info), dtype=np.int64, count=n)
    req_offs = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(counts, out=req_offs[1:])
    req_ids = _i32([r for t in tree_info for r in t.requests]) if req_offs[-1] else np.zeros(1, dtype=np.int32)
    ptrs = np.ascontiguousarray(np.asarray(KV_ptrs, dtype=np.int64))
    if ptrs.shape[0] != n + 1:
        raise FastTreePlannerError("KV_ptrs must have one entry per node plus one")
    splits, th1, th2 = _i32(list(KV_SPLIT_SIZES)[:2]), _i32(list(para_threshs1)[:2]), _i32(list(para_threshs2)[:2])
    tsq, tsk = _i32(list(TSQs)[:2]), _i32(list(TSKs)[:2])
    slot_map = None if kv_slot_map is None else _i32(kv_slot_map)
    handle = ctypes.c_void_p()
    rc = lib.ft_plan_create(
        n, _ptr32(parent), _ptr32(seqlen), _ptr32(children), req_offs.ctypes.data_as(_P64), _ptr32(req_ids),
        ptrs.ctypes.data_as(_P64), int(batch_size), int(num_kv_heads), _ptr32(splits), _ptr32(th1), _ptr32(th2),
        float(alpha), float(beta), float(gamma), _ptr32(tsq), _ptr32(tsk), int(kv_group_num),
        None if slot_map is None else _ptr32(slot_map), 0 if slot_map is None else slot_map.shape[0],
        ctypes.byref(handle))
    if rc != 0:
        raise FastTreePlannerError(f"ft_plan_create failed: {_ERRORS.get(rc, rc)}")
    try:
        out = []
        for which in range(N_ARRAYS):
            size = lib.ft_plan_size(handle, which)
            a = np.empty(max(size, 0), dtype=np.int32)
            rc = lib.ft_plan_copy(handle, which, _ptr32(a) if size else None, size)
            if rc != 0:
                raise FastTreePlannerError(f"ft_plan_copy failed: {_ERRORS.get(rc, rc)}")
            out.append(a)
        return out
    finally:
        lib.ft_plan_destroy(handle)
