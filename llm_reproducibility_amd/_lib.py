"""ctypes binding of libtbik_hip.so (declared in include/tbik_hip.h).

The library is the only compute path of this package: if it is missing, loading fails with an error
that says how to build it -- there is no eager / CPU fallback.
"""
from __future__ import annotations

import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libtbik_hip.so")

ABI_VERSION = 17
TBIK_OK = 0
TBIK_ERR_INVALID = 1
TBIK_ERR_ALIGNMENT = 2
TBIK_ERR_UNSUPPORTED = 3
TBIK_ERR_WORKSPACE = 4
TBIK_ERR_SCRATCH_LIMIT = 5
STATIC_SCRATCH_BYTES = 32 * 1024 * 1024

EXPORTS = (
    "tbik_abi_version", "tbik_error_string", "tbik_tree_params", "tbik_gemm_bf16", "tbik_gemm_workspace_bytes",
    "tbik_tree_combine_bf16", "tbik_tree_combine_f32",
    "bi_gemm_bf16", "bi_rmsnorm_bf16", "bi_log_softmax_workspace_bytes", "bi_log_softmax_f32", "bi_mean_dim", "bi_attention_bf16", "bi_silu_mul_bf16",
    "tbik_gemm_f16", "tbik_gemm_f16_workspace_bytes", "tbik_tree_combine_f16", "bi_gemm_f16", "tbik_gemm_f32", "bi_gemm_f32", "bi_rmsnorm_f16", "bi_silu_mul_f16", "bi_qk_norm_rope_cache_bf16", "bi_argmax_bf16",
    "tbik_gemm_bf16_static", "bi_log_softmax", "tbik_gemm_workspace_bytes_rowmajor_b", "tbik_gemm_plan_info",
    "bi_rmsnorm_gemm_bf16", "tbik_gemm_silu_mul_bf16", "bi_argmax_advance_bf16",
    "tbik_gemm_rmsnorm_bf16", "tbik_tree_combine_rmsnorm_bf16", "bi_attention_decode_qkv_bf16", "bi_gemm_silu_mul_bf16",
)

_lib = None


class TbikError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        msg = lib().tbik_error_string(code).decode()
        super().__init__(f"{where}: {msg} (code {code})")


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP kernels are the only implementation of this package. "
            "Build them with `python -m llm_reproducibility_amd.build` (needs hipcc).")
    L = ctypes.CDLL(LIB_PATH)
    i32, i64, vp, sz, f32 = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float
    pi32 = ctypes.POINTER(ctypes.c_int)
    L.tbik_abi_version.argtypes = []
    L.tbik_abi_version.restype = i32
    L.tbik_error_string.argtypes = [i32]
    L.tbik_error_string.restype = ctypes.c_char_p
    L.tbik_tree_params.argtypes = [i32, i32, pi32, pi32, pi32]
    L.tbik_tree_params.restype = i32
    L.tbik_gemm_bf16.argtypes = [vp, i64, vp, i64, i64, vp, i64, i32, i32, i32, i32, vp, vp, sz, vp]
    L.tbik_gemm_workspace_bytes.argtypes = [i32, i32, i32, i32]
    L.tbik_gemm_workspace_bytes.restype = sz
    L.tbik_gemm_bf16.restype = i32
    L.tbik_gemm_workspace_bytes_rowmajor_b.argtypes = [i32, i32, i32, i32, i32]
    L.tbik_gemm_workspace_bytes_rowmajor_b.restype = sz
    L.tbik_gemm_plan_info.argtypes = [i32, i32, i32, i32, i32, i32, ctypes.POINTER(ctypes.c_int)]
    L.tbik_gemm_plan_info.restype = i32
    L.tbik_tree_combine_bf16.argtypes = [ctypes.POINTER(vp), i32, vp, i64, vp]
    L.tbik_tree_combine_bf16.restype = i32
    L.bi_gemm_bf16.argtypes = [vp, i64, vp, i64, i64, vp, i64, i32, i32, i32, vp, vp]
    L.bi_gemm_bf16.restype = i32
    L.bi_rmsnorm_bf16.argtypes = [vp, i64, vp, i64, vp, vp, i64, vp, i64, i64, i32, f32, vp]
    L.bi_rmsnorm_bf16.restype = i32
    L.bi_log_softmax_workspace_bytes.argtypes = [i64, i64]
    L.bi_log_softmax_workspace_bytes.restype = sz
    L.bi_log_softmax_f32.argtypes = [vp, i64, vp, i64, i64, i64, vp, sz, i32, vp]
    L.bi_log_softmax_f32.restype = i32
    L.bi_log_softmax.argtypes = [vp, i64, i32, vp, i64, i32, i64, i64, vp, sz, i32, vp]
    L.bi_log_softmax.restype = i32
    L.bi_mean_dim.argtypes = [vp, vp, i64, i64, i64, i32, vp]
    L.bi_mean_dim.restype = i32
    L.tbik_gemm_f16.argtypes = L.tbik_gemm_bf16.argtypes
    L.tbik_gemm_f16.restype = i32
    L.tbik_gemm_f16_workspace_bytes.argtypes = [i32, i32, i32, i32]
    L.tbik_gemm_f16_workspace_bytes.restype = sz
    L.tbik_tree_combine_f16.argtypes = L.tbik_tree_combine_bf16.argtypes
    L.tbik_tree_combine_f16.restype = i32
    L.tbik_tree_combine_f32.argtypes = L.tbik_tree_combine_bf16.argtypes
    L.tbik_tree_combine_f32.restype = i32
    L.bi_gemm_f16.argtypes = L.bi_gemm_bf16.argtypes
    L.bi_gemm_f16.restype = i32
    L.tbik_gemm_f32.argtypes = [vp, i64, vp, i64, i64, vp, i64, i32, i32, i32, i32, vp, vp]
    L.tbik_gemm_f32.restype = i32
    L.bi_gemm_f32.argtypes = [vp, i64, vp, i64, i64, vp, i64, i32, i32, i32, vp, vp]
    L.bi_gemm_f32.restype = i32
    L.bi_silu_mul_bf16.argtypes = [vp, i64, vp, i64, i64, i32, vp]
    L.bi_silu_mul_bf16.restype = i32
    L.bi_rmsnorm_f16.argtypes = L.bi_rmsnorm_bf16.argtypes
    L.bi_rmsnorm_f16.restype = i32
    L.bi_silu_mul_f16.argtypes = L.bi_silu_mul_bf16.argtypes
    L.bi_silu_mul_f16.restype = i32
    L.bi_qk_norm_rope_cache_bf16.argtypes = [vp, i64, vp, vp, vp, vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, i32, f32, vp]
    L.bi_qk_norm_rope_cache_bf16.restype = i32
    L.bi_argmax_bf16.argtypes = [vp, i64, vp, i64, i32, vp]
    L.bi_argmax_bf16.restype = i32
    L.bi_argmax_advance_bf16.argtypes = [vp, i64, vp, i64, i32, vp, i64, vp, vp, vp, vp]
    L.bi_argmax_advance_bf16.restype = i32
    L.bi_attention_decode_qkv_bf16.argtypes = [vp, i64, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, f32, f32, vp]
    L.bi_attention_decode_qkv_bf16.restype = i32
    L.bi_gemm_silu_mul_bf16.argtypes = [vp, i64, vp, i64, vp, i64, i32, i32, i32, vp]
    L.bi_gemm_silu_mul_bf16.restype = i32
    L.tbik_gemm_rmsnorm_bf16.argtypes = [vp, i64, vp, i64, i64, i32, i32, i32, i32, vp, vp, i64, vp, ctypes.c_float, vp, i64, vp, i64,
                                         vp, ctypes.c_size_t, vp]
    L.tbik_gemm_rmsnorm_bf16.restype = i32
    L.tbik_tree_combine_rmsnorm_bf16.argtypes = [ctypes.POINTER(vp), i32, i64, i32, vp, vp, i64, vp, ctypes.c_float, vp, i64, vp, i64, vp]
    L.tbik_tree_combine_rmsnorm_bf16.restype = i32
    L.tbik_gemm_bf16_static.argtypes = [vp, i64, vp, i64, i64, vp, i64, i32, i32, i32, i32, vp, vp]
    L.tbik_gemm_bf16_static.restype = i32
    L.bi_rmsnorm_gemm_bf16.argtypes = [vp, i64, vp, i64, vp, f32, vp, i64, vp, i64, i64, vp, i64, i32, i32, i32, vp, vp]
    L.bi_rmsnorm_gemm_bf16.restype = i32
    L.tbik_gemm_silu_mul_bf16.argtypes = [vp, vp, i64, vp, i64, i64, vp, i64, i32, i32, i32, i32, vp, vp]
    L.tbik_gemm_silu_mul_bf16.restype = i32
    L.bi_attention_bf16.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, vp]
    L.bi_attention_bf16.restype = i32
    if L.tbik_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH}: ABI version {L.tbik_abi_version()} does not match this package ({ABI_VERSION})")
    _lib = L
    return L


def check(code: int, where: str) -> None:
    if code != TBIK_OK:
        raise TbikError(code, where)


def tree_params(K: int, leaf_k: int):
    """(T, FLB, LEVEL_K) of a K extent; ValueError if K is not a whole number of leaves."""
    t, f, l = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    rc = lib().tbik_tree_params(int(K), int(leaf_k), ctypes.byref(t), ctypes.byref(f), ctypes.byref(l))
    if rc != TBIK_OK:
        raise ValueError(f"K={K} is not a whole number of leaves of {leaf_k}")
    return t.value, f.value, l.value
