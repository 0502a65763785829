"""ctypes binding of libfasttree_hip.so (the C ABI declared in include/fasttree_hip.h).

There is no fallback: if the library has not been built, or a call returns an error
code, this module raises.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

LIB_NAME = "libfasttree_hip.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

FT_DTYPE_F16 = 0
FT_DTYPE_BF16 = 1

FT_ERR_HEAD_DIM = -3

_I64x6 = [c_int64] * 6
_P = c_void_p

SIGNATURES = {
    "ft_version": (c_char_p, []),
    "ft_error_string": (c_char_p, [c_int]),
    "ft_static_scratch_bytes": (c_int64, []),
    "ft_stage1": (c_int, [_P, _P, _P] + _I64x6 + [_P] * 6 + [c_int] * 7 + [c_float]
                  + [_P, c_int64, c_int64, _P, c_int64, c_int, _P]),
    "ft_stage1_phases": (c_int, [_P, _P, _P] + _I64x6 + [_P] * 6 + [_P, c_int64, c_int64, _P, c_int64] + [_P] * 4
                         + [c_int] * 3 + [c_float, c_int, _P]),
    "ft_stage2": (c_int, [_P, _P, _P, _P, c_int64, c_int64, _P, c_int64, _P, c_int64, c_int64,
                          c_int, c_int, c_int, c_int, _P]),
    "ft_decode": (c_int, [_P, _P, _P, _P] + [c_int64] * 8 + [_P] * 9
                  + [_P, c_int64, c_int64, _P, c_int64] + [_P] * 4 + [c_int] * 4 + [c_float, c_int, _P]),
    "ft_stage1_programs": (c_int, [_P, _P, _P] + _I64x6 + [_P] * 6 + [_P, c_int64, c_int64, _P, c_int64] + [_P] * 2
                           + [_P, c_int, c_int, _P, _P] + [c_int] * 3 + [c_float, c_int, _P]),
    "ft_decode_programs": (c_int, [_P, _P, _P, _P] + [c_int64] * 8 + [_P] * 9
                           + [_P, c_int64, c_int64, _P, c_int64] + [_P] * 2 + [_P, c_int, c_int, _P, _P, _P] + [c_int] * 4
                           + [c_float, c_int, _P]),
    "ft_decode_static": (c_int, [_P, _P, _P, _P] + [c_int64] * 8 + [_P] * 9 + [c_int64] + [_P] * 2
                         + [_P, c_int, c_int, _P, _P, _P] + [c_int] * 4 + [c_float, c_int, _P]),
    "ft_deft_stage1": (c_int, [_P, _P, _P] + _I64x6 + [_P] * 6 + [_P, _P] + [c_int] * 5 + [c_float]
                       + [_P, c_int64, c_int64, _P, c_int64, c_int, _P]),
    "ft_deft_decode": (c_int, [_P, _P, _P, _P] + [c_int64] * 8 + [_P] * 6 + [_P, _P] + [_P] * 3
                       + [_P, c_int64, c_int64, _P, c_int64] + [c_int] * 6 + [c_float, c_int, _P]),
    "ft_gathered_decode": (c_int, [_P, _P, _P, _P, _P] + [c_int64] * 4 + [c_int] * 6 + [c_float]
                           + [_P, _P, c_int, _P]),
    "ft_store_kv": (c_int, [_P, _P] + [c_int64] * 4 + [_P, c_int, c_int, _P, _P] + [c_int64] * 5
                    + [c_int, c_int, c_int, _P]),
}

_lib = None


class FastTreeLibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the shared library once and attach the argument types."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FastTreeLibraryError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc --offload-arch=gfx950). There is no fallback path."
        )
    # torch ships its own HIP runtime with the same SONAME; importing it first makes the
    # dynamic loader reuse that copy, so streams and pointers are shared with torch.
    import torch  # noqa: F401

    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code == 0:
        return
    msg = load().ft_error_string(code).decode()
    if code == FT_ERR_HEAD_DIM:
        # the reference asserts on the head dimension (kernel_bench/fasttree.py:437-439)
        raise AssertionError(f"{what}: {msg}")
    raise FastTreeLibraryError(f"{what}: {msg} (code {code})")


def int32_pair(values):
    if len(values) != 2:
        raise ValueError("expected a sequence of two integers")
    return (c_int32 * 2)(int(values[0]), int(values[1]))
