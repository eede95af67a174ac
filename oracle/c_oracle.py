"""ctypes binding of oracle/libtbik_oracle.so (test infrastructure only)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtbik_oracle.so")


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "tbik_oracle.c")):
        subprocess.run(["make", "-C", _HERE, "-B", "libtbik_oracle.so"], check=True, capture_output=True)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        _lib.tbik_oracle_matmul_tree.argtypes = [vp, i64, vp, i64, i64, vp, i64, ci, ci, ci, ci, vp]
        _lib.tbik_oracle_matmul_tree.restype = ci
        _lib.tbik_oracle_tree_combine.argtypes = [ctypes.POINTER(vp), ci, vp, i64]
        _lib.tbik_oracle_tree_combine.restype = ci
        _lib.tbik_oracle_tree_params.argtypes = [ci, ci] + [ctypes.POINTER(ci)] * 3
        _lib.tbik_oracle_tree_params.restype = ci
    return _lib


def tree_params(K: int, leaf: int):
    t, f, l = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    rc = lib().tbik_oracle_tree_params(K, leaf, ctypes.byref(t), ctypes.byref(f), ctypes.byref(l))
    if rc:
        raise ValueError("K is not a whole number of leaves")
    return t.value, f.value, l.value


def matmul_tree(A: torch.Tensor, B: torch.Tensor, bias=None, leaf: int = 256) -> torch.Tensor:
    assert A.dtype == torch.bfloat16 and B.dtype == torch.bfloat16 and A.stride(1) == 1
    M, K = A.shape
    N = B.shape[1]
    C = torch.empty((M, N), dtype=torch.bfloat16)
    rc = lib().tbik_oracle_matmul_tree(A.data_ptr(), A.stride(0), B.data_ptr(), B.stride(0), B.stride(1),
                                       C.data_ptr(), C.stride(0), M, N, K, leaf,
                                       None if bias is None else bias.data_ptr())
    assert rc == 0, rc
    return C


def tree_combine(parts) -> torch.Tensor:
    parts = [p.contiguous() for p in parts]
    out = torch.empty_like(parts[0])
    arr = (ctypes.c_void_p * len(parts))(*[p.data_ptr() for p in parts])
    rc = lib().tbik_oracle_tree_combine(arr, len(parts), out.data_ptr(), out.numel())
    if rc:
        raise ValueError("the number of partials must be a power of two")
    return out
