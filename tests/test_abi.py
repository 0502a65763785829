"""The C-ABI library loads and exports every symbol the header declares; argument checks
that run before any device work return the documented codes (CPU only, no compute)."""

import ctypes
import os
import re

import pytest

from fasttree_hip import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fasttree_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ft_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = declared_symbols()
    assert names == ["ft_decode", "ft_decode_programs", "ft_decode_static", "ft_deft_decode", "ft_deft_stage1", "ft_error_string", "ft_gathered_decode", "ft_stage1",
                     "ft_stage1_phases", "ft_stage1_programs", "ft_stage2", "ft_static_scratch_bytes", "ft_store_kv", "ft_version"]
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), name
    assert set(_lib.SIGNATURES) == set(names)


def test_version_and_error_strings():
    lib = _lib.load()
    assert b"gfx950" in lib.ft_version()
    assert lib.ft_error_string(0) == b"ok"
    for code in range(-7, 0):
        assert lib.ft_error_string(code) not in (b"ok", b"unknown error")
    assert lib.ft_error_string(-99) == b"unknown error"
    assert lib.ft_static_scratch_bytes() == 64 << 20


def test_argument_checks_return_codes_without_touching_a_device():
    lib = _lib.load()
    null = None
    base = dict(head_dim=128, g=4, dtype=0)

    def stage1(head_dim=128, g=4, dtype=0, count=1, ptr=null, sm_scale=0.1, stride=1024):
        return lib.ft_stage1(ptr, ptr, ptr, stride, 128, stride, 128, stride, 128, ptr, ptr, ptr, ptr, ptr, ptr,
                             0, count, 8, g, head_dim, 16, 32, sm_scale, ptr, 4096, 128, ptr, 32, dtype, None)

    assert stage1(head_dim=48) == -3          # FT_ERR_HEAD_DIM
    assert stage1(head_dim=8) == -3
    assert stage1(head_dim=16) == -1          # a head dimension the reference takes too (kernel_bench/fasttree.py:439)
    assert stage1(dtype=7) == -2              # FT_ERR_DTYPE
    assert stage1(g=0) == -4                  # FT_ERR_GROUP
    assert stage1(count=0) == 0               # nothing to do is not an error
    assert stage1() == -1                     # FT_ERR_NULL_POINTER
    assert stage1(ptr=0x1000, sm_scale=0.0) == -6
    assert stage1(ptr=0x1004) == -5           # FT_ERR_ALIGNMENT (pointer)
    assert stage1(ptr=0x1000, stride=1001) == -5
    with pytest.raises(AssertionError):
        _lib.check(-3, "x")
    with pytest.raises(_lib.FastTreeLibraryError):
        _lib.check(-5, "x")

    def store(ptr=0x1000, tokens=3, head_dim=128, dtype=0, stride=1024, heads=8):
        return lib.ft_store_kv(ptr, ptr, stride, 128, stride, 128, ptr, 0, tokens, ptr, ptr, stride, 128, stride, 128,
                               100, heads, head_dim, dtype, None)

    assert store(tokens=0) == 0
    assert store(ptr=null) == -1
    assert store(dtype=3) == -2
    assert store(head_dim=12) == -3
    assert store(ptr=0x1008) == -5
    assert store(stride=1028) == -5
    assert store(tokens=-1) == -6 and store(heads=0) == -6 and store(stride=-1024) == -6


def test_decode_refuses_cpu_tensors():
    import torch
    from fasttree_hip.decode import fasttree_decode

    q = torch.zeros(1, 4, 32, dtype=torch.float16)
    idx = torch.zeros(40, dtype=torch.int32)
    with pytest.raises(_lib.FastTreeLibraryError):
        fasttree_decode(q, q, q, q, idx, idx, idx, idx, idx, idx, idx, idx, idx, q.float(), q.float()[..., 0],
                        [0, 1], [0, 0], [16, 4], [32, 32], 0.1)
    with pytest.raises(AssertionError):   # mismatched q / k head dimension, as the reference asserts
        fasttree_decode(q, q[..., :16], q, q, idx, idx, idx, idx, idx, idx, idx, idx, idx, q.float(), q.float()[..., 0],
                        [0, 1], [0, 0], [16, 4], [32, 32], 0.1)


def test_planner_header_symbols_are_exported():
    from fasttree_hip import _plan_lib
    text = open(os.path.join(ROOT, "include", "fasttree_plan.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(ft_plan_[a-z0-9_]+)\s*\(", text)))
    assert names == ["ft_plan_copy", "ft_plan_create", "ft_plan_destroy", "ft_plan_size", "ft_plan_version"]
    lib = ctypes.CDLL(_plan_lib.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), name
    assert set(_plan_lib.SIGNATURES) == set(names)
    # the enum of result arrays and the Python constants agree
    enum = re.search(r"enum \{\s*FT_PLAN_KV_ENTRIES = 0,(.*?)FT_PLAN_ARRAYS", text, flags=re.S).group(1)
    assert len(re.findall(r"FT_PLAN_[A-Z_]+", enum)) + 1 == _plan_lib.N_ARRAYS
    assert _plan_lib.load().ft_plan_size(None, 0) == -1
