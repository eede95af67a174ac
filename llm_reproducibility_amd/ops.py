"""Torch custom ops over the C ABI of libtbik_hip.so.

Each op allocates its output with torch, passes raw device pointers, element strides and the current
HIP stream to one `extern "C"` entry point, and raises on a non-zero return code.  The ops are
registered as `torch.ops.tbik.*` for the GPU device type only; there is no CPU path, CPU tensors raise.

Eager callers reach the same implementation function directly (the dispatcher round trip of a Python
custom op costs ~10 us per call, more than most of these kernels take); under torch.compile the
registered op is used so the call stays a single opaque node.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """The current stream of the tensor's device as a raw handle.  The private accessor (the one torch's own compiled code
    uses) returns the handle without building a Stream object: 0.3 us instead of 3 us of host time per launch."""
    if _raw_stream is not None and t.device.index is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("tbik ops run on the GPU only (HIP kernels); got a tensor on " + str(t.device))


def _aligned16(t: torch.Tensor) -> bool:
    return t.data_ptr() % 16 == 0


def _is_f16(*tensors) -> bool:
    """True for float16 operands, False for bfloat16; every operand must have the same one of the two."""
    dts = {t.dtype for t in tensors if t is not None}
    if len(dts) != 1 or not dts <= {torch.bfloat16, torch.float16}:
        raise NotImplementedError(f"16-bit GEMM kernels take all-bfloat16 or all-float16 operands, got {sorted(map(str, dts))}")
    return dts == {torch.float16}


def _rows_f32(t: torch.Tensor):
    """fp32 operand with a contiguous last dim, 16-byte aligned rows (leading dimension a multiple of 4)."""
    ok = t.stride(1) == 1 and _aligned16(t) and (t.shape[0] == 1 or (t.stride(0) >= t.shape[1] and t.stride(0) % 4 == 0))
    if ok:
        return t, (t.shape[1] if t.shape[0] == 1 else t.stride(0))
    c = t.contiguous()
    if not _aligned16(c) or c.shape[1] % 4 != 0:
        c = torch.nn.functional.pad(c, (0, (-c.shape[1]) % 4))[:, : t.shape[1]] if c.shape[1] % 4 else c.clone()
    return c, c.stride(0)


def _gemm_f32(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor], leaf_k: int, tree: bool) -> torch.Tensor:
    M, K = A.shape
    N = B.shape[1]
    if K % 16 != 0:  # only the single-accumulator form gets here: zero columns do not change a sequential sum
        pad = (-K) % 16
        A = torch.nn.functional.pad(A, (0, pad))
        B = torch.nn.functional.pad(B, (0, 0, 0, pad))
        K += pad
    a, lda = _rows_f32(A)
    w, ldw = _rows_f32(B.t())
    b = None if bias is None else bias.contiguous()
    C = torch.empty((M, N), device=A.device, dtype=torch.float32)
    L = _lib.lib()
    if tree:
        rc = L.tbik_gemm_f32(a.data_ptr(), lda, w.data_ptr(), 1, ldw, C.data_ptr(), C.stride(0), M, N, K, leaf_k,
                             None if b is None else b.data_ptr(), _stream(A))
    else:
        rc = L.bi_gemm_f32(a.data_ptr(), lda, w.data_ptr(), 1, ldw, C.data_ptr(), C.stride(0), M, N, K,
                           None if b is None else b.data_ptr(), _stream(A))
    _lib.check(rc, "tbik_gemm_f32" if tree else "bi_gemm_f32")
    return C


def _rows16(t: torch.Tensor):
    """(tensor, leading dimension) with a contiguous last dim and 16-byte aligned rows; copies if needed."""
    ok = t.stride(1) == 1 and _aligned16(t) and t.shape[1] % 8 == 0
    if ok and t.shape[0] == 1:
        return t, t.shape[1]
    if ok and t.stride(0) >= t.shape[1] and t.stride(0) % 8 == 0:
        return t, t.stride(0)
    c = t.contiguous()
    if not _aligned16(c):
        c = c.clone()
    return c, c.shape[1]


# Rows from which a row-major [K,N] operand is repacked into the native [N,K] layout instead of being consumed in
# place.  In place it runs on the 64-row tiled kernels only (the pipelines with 128x256 tiles are built for [N,K]), so
# the time grows with the rows; a repack costs one transposing copy of B (60 us for 4096 x 4096, 180 us for
# 12288 x 4096 with the library's copy kernel) and then the fast kernels.  Measured on MI355X, bf16, B of 4096 x 4096 /
# 12288 x 4096 / 4096 x 12288: the tree matmul in place wins up to 512 rows (74 / 199 / 197 us against 93 / 244 / 256)
# and loses from 1024 on (133 / 382 / 393 against 110 / 305 / 303; at 4096 rows 523 / 1523 / 1567 against 205 / 594 /
# 622); the single-accumulator mm, which cannot cut K, wins up to 1024 rows and loses from 2048 on (148 / 416 / 437
# against 120 / 335 / 332).  Same bits either way.
_REPACK_ROWS_TREE = 1024
_REPACK_ROWS_MM = 2048


def _weight_operand(B: torch.Tensor, rows: int = 0, tree: bool = True):
    """How a [K,N] operand is handed to the kernels: (tensor whose data_ptr is passed, ldb_k, ldb_n).

    `weight.t()` of an nn.Linear weight ([N,K], K contiguous) is the native layout (ldb_k = 1), used without a copy; a
    row-major [K,N] operand (N contiguous: a plain `x @ B`) is consumed in place too (ldb_n = 1) unless the product has
    so many rows (`rows`) that a repack into the native layout pays.  Anything else -- neither dimension contiguous,
    rows not 16-byte aligned -- is repacked as well."""
    K, N = B.shape
    if B.stride(0) == 1 and _aligned16(B) and K % 8 == 0 and (N == 1 or (B.stride(1) >= K and B.stride(1) % 8 == 0)):
        return B, 1, (K if N == 1 else B.stride(1))
    in_place = rows < (_REPACK_ROWS_TREE if tree else _REPACK_ROWS_MM)
    if in_place and B.stride(1) == 1 and _aligned16(B) and B.stride(0) >= N and B.stride(0) % 8 == 0:
        return B, B.stride(0), 1
    w, ldw = _rows16(B.t())
    return w, 1, ldw


# --------------------------------------------------------------------------------------------
# tree-ordered GEMM
# --------------------------------------------------------------------------------------------
def _gemm_tree_impl(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor], leaf_k: int) -> torch.Tensor:
    _require_gpu(A, B, bias)
    if A.dtype == torch.float32 and B.dtype == torch.float32 and (bias is None or bias.dtype == torch.float32):
        return _gemm_f32(A, B, bias, leaf_k, True)
    M, K = A.shape
    N = B.shape[1]
    a, lda = _rows16(A)
    w, ldb_k, ldb_n = _weight_operand(B, M, True)
    b = None if bias is None else bias.contiguous()
    f16 = _is_f16(A, B, bias)
    C = torch.empty((M, N), device=A.device, dtype=A.dtype)
    L = _lib.lib()
    if ldb_k != 1:
        ws_bytes = L.tbik_gemm_workspace_bytes_rowmajor_b(M, N, K, leaf_k, int(f16))
    else:
        ws_bytes = (L.tbik_gemm_f16_workspace_bytes if f16 else L.tbik_gemm_workspace_bytes)(M, N, K, leaf_k)
    ws = torch.empty(ws_bytes, device=A.device, dtype=torch.uint8) if ws_bytes else None
    rc = (L.tbik_gemm_f16 if f16 else L.tbik_gemm_bf16)(a.data_ptr(), lda, w.data_ptr(), ldb_k, ldb_n, C.data_ptr(), C.stride(0),
                          M, N, K, leaf_k, None if b is None else b.data_ptr(),
                          None if ws is None else ws.data_ptr(), ws_bytes, _stream(A))
    _lib.check(rc, "tbik_gemm_bf16")
    return C


_gemm_tree_op = torch.library.custom_op("tbik::gemm_tree", _gemm_tree_impl, mutates_args=(), device_types="cuda")


def gemm_tree(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor], leaf_k: int) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return _gemm_tree_op(A, B, bias, leaf_k)
    return _gemm_tree_impl(A, B, bias, leaf_k)


@_gemm_tree_op.register_fake
def _(A, B, bias, leaf_k):
    return A.new_empty((A.shape[0], B.shape[1]))


def _tree_combine_impl(parts: List[torch.Tensor]) -> torch.Tensor:
    _require_gpu(*parts)
    ps = [p.contiguous() for p in parts]
    out = torch.empty_like(ps[0])
    arr = (ctypes.c_void_p * len(ps))(*[p.data_ptr() for p in ps])
    L = _lib.lib()
    if ps[0].dtype == torch.float32:
        if any(p.dtype != torch.float32 for p in ps):
            raise NotImplementedError("tree_combine takes partials of one dtype")
        fn = L.tbik_tree_combine_f32
    else:
        fn = L.tbik_tree_combine_f16 if _is_f16(*ps) else L.tbik_tree_combine_bf16
    rc = fn(arr, len(ps), out.data_ptr(), out.numel(), _stream(out))
    _lib.check(rc, "tbik_tree_combine")
    return out


_tree_combine_op = torch.library.custom_op("tbik::tree_combine", _tree_combine_impl, mutates_args=(), device_types="cuda")


def tree_combine(parts: List[torch.Tensor]) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return _tree_combine_op(parts)
    return _tree_combine_impl(parts)


@_tree_combine_op.register_fake
def _(parts):
    return torch.empty_like(parts[0])


# --------------------------------------------------------------------------------------------
# batch-invariant ops
# --------------------------------------------------------------------------------------------
def _bi_gemm_impl(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    _require_gpu(A, B, bias)
    if A.dtype == torch.float32 and B.dtype == torch.float32 and (bias is None or bias.dtype == torch.float32):
        return _gemm_f32(A, B, bias, 0, False)
    M, K = A.shape
    N = B.shape[1]
    if K % 8 != 0:
        # zero columns do not change a sequential fp32 accumulation
        pad = (-K) % 8
        A = torch.nn.functional.pad(A, (0, pad))
        B = torch.nn.functional.pad(B, (0, 0, 0, pad))
        K += pad
    a, lda = _rows16(A)
    w, ldb_k, ldb_n = _weight_operand(B, M, False)
    b = None if bias is None else bias.contiguous()
    C = torch.empty((M, N), device=A.device, dtype=A.dtype)
    L = _lib.lib()
    rc = (L.bi_gemm_f16 if _is_f16(A, B, bias) else L.bi_gemm_bf16)(a.data_ptr(), lda, w.data_ptr(), ldb_k, ldb_n, C.data_ptr(), C.stride(0),
                                 M, N, K, None if b is None else b.data_ptr(), _stream(A))
    _lib.check(rc, "bi_gemm")
    return C


_bi_gemm_op = torch.library.custom_op("tbik::bi_gemm", _bi_gemm_impl, mutates_args=(), device_types="cuda")


def bi_gemm(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return _bi_gemm_op(A, B, bias)
    return _bi_gemm_impl(A, B, bias)


@_bi_gemm_op.register_fake
def _(A, B, bias):
    return A.new_empty((A.shape[0], B.shape[1]))


def _bi_rmsnorm_impl(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    _require_gpu(x, weight)
    hidden = x.shape[-1]
    x2, ldx = _rows16(x.reshape(-1, hidden))
    out = torch.empty((x2.shape[0], hidden), device=x.device, dtype=x.dtype)
    w = None if weight is None else weight.contiguous()
    L = _lib.lib()
    rc = (L.bi_rmsnorm_f16 if _is_f16(x, weight) else L.bi_rmsnorm_bf16)(x2.data_ptr(), ldx, None, 0, None if w is None else w.data_ptr(),
                                    out.data_ptr(), out.stride(0), None, 0, x2.shape[0], hidden, eps, _stream(x))
    _lib.check(rc, "bi_rmsnorm")
    return out.reshape(x.shape)


_bi_rmsnorm_op = torch.library.custom_op("tbik::bi_rmsnorm", _bi_rmsnorm_impl, mutates_args=(), device_types="cuda")


def bi_rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return _bi_rmsnorm_op(x, weight, eps)
    return _bi_rmsnorm_impl(x, weight, eps)


@_bi_rmsnorm_op.register_fake
def _(x, weight, eps):
    return torch.empty_like(x)


def _bi_add_rmsnorm_impl(x: torch.Tensor, residual: torch.Tensor, weight: Optional[torch.Tensor],
                        eps: float) -> List[torch.Tensor]:
    _require_gpu(x, residual, weight)
    hidden = x.shape[-1]
    x2, ldx = _rows16(x.reshape(-1, hidden))
    r2, ldr = _rows16(residual.reshape(-1, hidden))
    out = torch.empty((x2.shape[0], hidden), device=x.device, dtype=x.dtype)
    rout = torch.empty_like(out)
    w = None if weight is None else weight.contiguous()
    L = _lib.lib()
    rc = (L.bi_rmsnorm_f16 if _is_f16(x, residual, weight) else L.bi_rmsnorm_bf16)(x2.data_ptr(), ldx, r2.data_ptr(), ldr,
                                    None if w is None else w.data_ptr(), out.data_ptr(), out.stride(0),
                                    rout.data_ptr(), rout.stride(0), x2.shape[0], hidden, eps, _stream(x))
    _lib.check(rc, "bi_rmsnorm")
    return [out.reshape(x.shape), rout.reshape(x.shape)]


_bi_add_rmsnorm_op = torch.library.custom_op("tbik::bi_add_rmsnorm", _bi_add_rmsnorm_impl, mutates_args=(), device_types="cuda")


def bi_add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, weight: Optional[torch.Tensor],
                        eps: float) -> List[torch.Tensor]:
    if torch.compiler.is_compiling():
        return _bi_add_rmsnorm_op(x, residual, weight, eps)
    return _bi_add_rmsnorm_impl(x, residual, weight, eps)


@_bi_add_rmsnorm_op.register_fake
def _(x, residual, weight, eps):
    return [torch.empty_like(x), torch.empty_like(x)]


def _bi_log_softmax_impl(x: torch.Tensor, write_softmax: bool, to_float: bool) -> torch.Tensor:
    """log_softmax (or softmax) over the last dimension of an fp32 / bf16 / fp16 tensor, in the input's dtype or,
    with `to_float`, in fp32; the kernel reads the input dtype itself."""
    _require_gpu(x)
    if x.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"bi_log_softmax: unsupported dtype {x.dtype}")
    cols = x.shape[-1]
    x2 = x.reshape(-1, cols)
    if x2.stride(1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < cols):
        x2 = x2.contiguous()
    rows = x2.shape[0]
    out_dtype = torch.float32 if to_float else x.dtype
    out = torch.empty((rows, cols), device=x.device, dtype=out_dtype)
    L = _lib.lib()
    nws = L.bi_log_softmax_workspace_bytes(rows, cols)
    ws = torch.empty((nws + 3) // 4, device=x.device, dtype=torch.float32) if nws else None
    rc = L.bi_log_softmax(x2.data_ptr(), x2.stride(0) if rows > 1 else cols, _DTYPE_CODE[x.dtype], out.data_ptr(),
                          out.stride(0), _DTYPE_CODE[out_dtype], rows, cols, None if ws is None else ws.data_ptr(), nws,
                          int(write_softmax), _stream(x))
    _lib.check(rc, "bi_log_softmax")
    return out.reshape(x.shape)


_bi_log_softmax_op = torch.library.custom_op("tbik::bi_log_softmax", _bi_log_softmax_impl, mutates_args=(), device_types="cuda")


def bi_log_softmax(x: torch.Tensor, write_softmax: bool, to_float: bool = False) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return _bi_log_softmax_op(x, write_softmax, to_float)
    return _bi_log_softmax_impl(x, write_softmax, to_float)


@_bi_log_softmax_op.register_fake
def _(x, write_softmax, to_float):
    return torch.empty_like(x, dtype=torch.float32 if to_float else x.dtype)


def bi_log_softmax_f32(x: torch.Tensor, write_softmax: bool) -> torch.Tensor:
    """fp32 in, fp32 out (kept for callers of the earlier name)."""
    return bi_log_softmax(x.float(), write_softmax)


def _bi_mean_dim_impl(x: torch.Tensor, dim: int, keepdim: bool) -> torch.Tensor:
    _require_gpu(x)
    if x.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"bi_mean_dim: unsupported dtype {x.dtype}")
    dim = dim % x.ndim
    shape = list(x.shape)
    outer = 1
    for s in shape[:dim]:
        outer *= s
    n = shape[dim]
    inner = 1
    for s in shape[dim + 1:]:
        inner *= s
    xc = x.contiguous()
    out_shape = shape[:dim] + ([1] if keepdim else []) + shape[dim + 1:]
    out = torch.empty(out_shape, device=x.device, dtype=x.dtype)
    rc = _lib.lib().bi_mean_dim(xc.data_ptr(), out.data_ptr(), outer, n, inner, _DTYPE_CODE[x.dtype], _stream(x))
    _lib.check(rc, "bi_mean_dim")
    return out


_bi_mean_dim_op = torch.library.custom_op("tbik::bi_mean_dim", _bi_mean_dim_impl, mutates_args=(), device_types="cuda")


def bi_mean_dim(x: torch.Tensor, dim: int, keepdim: bool) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return _bi_mean_dim_op(x, dim, keepdim)
    return _bi_mean_dim_impl(x, dim, keepdim)


@_bi_mean_dim_op.register_fake
def _(x, dim, keepdim):
    dim = dim % x.ndim
    shape = list(x.shape)
    out_shape = shape[:dim] + ([1] if keepdim else []) + shape[dim + 1:]
    return x.new_empty(out_shape)


# --------------------------------------------------------------------------------------------
# fixed-order attention
# --------------------------------------------------------------------------------------------
def _bi_attention_bf16_impl(q: torch.Tensor, k_cache: torch.Tensor, vt_cache: torch.Tensor, q_start: torch.Tensor,
                            q_len: torch.Tensor, ctx_len: torch.Tensor, max_q_len: int, scale: float) -> torch.Tensor:
    _require_gpu(q, k_cache, vt_cache, q_start, q_len, ctx_len)
    tokens, q_heads, head_dim = q.shape
    batch, kv_heads, max_len, _ = k_cache.shape
    assert vt_cache.shape == (batch, kv_heads, head_dim, max_len)
    assert q.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and vt_cache.dtype == torch.bfloat16
    assert q_start.dtype == torch.int32 and q_len.dtype == torch.int32 and ctx_len.dtype == torch.int32
    q = q.contiguous()
    assert k_cache.is_contiguous() and vt_cache.is_contiguous()
    out = torch.empty_like(q)
    rc = _lib.lib().bi_attention_bf16(q.data_ptr(), k_cache.data_ptr(), vt_cache.data_ptr(), out.data_ptr(),
                                      q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(), batch, max_q_len,
                                      q_heads, kv_heads, head_dim, max_len, scale, _stream(q))
    _lib.check(rc, "bi_attention_bf16")
    return out


_bi_attention_bf16_op = torch.library.custom_op("tbik::bi_attention_bf16", _bi_attention_bf16_impl, mutates_args=(),
                                                device_types="cuda")


def bi_attention_bf16(q: torch.Tensor, k_cache: torch.Tensor, vt_cache: torch.Tensor, q_start: torch.Tensor,
                      q_len: torch.Tensor, ctx_len: torch.Tensor, max_q_len: int, scale: float) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return _bi_attention_bf16_op(q, k_cache, vt_cache, q_start, q_len, ctx_len, max_q_len, scale)
    return _bi_attention_bf16_impl(q, k_cache, vt_cache, q_start, q_len, ctx_len, max_q_len, scale)


@_bi_attention_bf16_op.register_fake
def _(q, k_cache, vt_cache, q_start, q_len, ctx_len, max_q_len, scale):
    return torch.empty_like(q)


# --------------------------------------------------------------------------------------------
# gated activation in front of down_proj
# --------------------------------------------------------------------------------------------
def _bi_silu_mul_impl(gate_up: torch.Tensor) -> torch.Tensor:
    _require_gpu(gate_up)
    f16 = _is_f16(gate_up)
    two_i = gate_up.shape[-1]
    if two_i % 16 != 0:
        raise ValueError(f"bi_silu_mul: last dimension {two_i} must be a multiple of 16")
    inter = two_i // 2
    g2, ld = _rows16(gate_up.reshape(-1, two_i))
    out = torch.empty((g2.shape[0], inter), device=gate_up.device, dtype=gate_up.dtype)
    L = _lib.lib()
    rc = (L.bi_silu_mul_f16 if f16 else L.bi_silu_mul_bf16)(g2.data_ptr(), ld, out.data_ptr(), out.stride(0), g2.shape[0], inter, _stream(gate_up))
    _lib.check(rc, "bi_silu_mul")
    return out.reshape(*gate_up.shape[:-1], inter)


_bi_silu_mul_op = torch.library.custom_op("tbik::bi_silu_mul", _bi_silu_mul_impl, mutates_args=(), device_types="cuda")


def bi_silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """act = silu(gate_up[..., :I]) * gate_up[..., I:] (I = half the last dimension), fused, bf16."""
    if torch.compiler.is_compiling():
        return _bi_silu_mul_op(gate_up)
    return _bi_silu_mul_impl(gate_up)


@_bi_silu_mul_op.register_fake
def _(gate_up):
    return gate_up.new_empty((*gate_up.shape[:-1], gate_up.shape[-1] // 2))


# --------------------------------------------------------------------------------------------
# one-launch compositions for decode-sized batches (bit-identical to the two-launch forms they fall back to)
# --------------------------------------------------------------------------------------------
# Shapes for which a one-launch entry point answered 'unsupported': whether it applies depends on the shape alone, so the
# next call of the same shape goes to the separate calls at once (no output allocated for a call that will not run).
_declined: set = set()


def rmsnorm_gemm(x: torch.Tensor, norm_weight: Optional[torch.Tensor], eps: float, residual: Optional[torch.Tensor],
                 B: torch.Tensor, bias: Optional[torch.Tensor] = None):
    """(bi_gemm(rms_norm(x [+ residual]) * norm_weight, B) (+ bias), new residual or None).

    One launch (`bi_rmsnorm_gemm_bf16`: the matmul normalises the activations while it stages them) for a few bf16 rows
    against an nn.Linear weight handed over as `weight.t()`; the two launches otherwise.  Same bits either way."""
    _require_gpu(x, norm_weight, residual, B, bias)
    M, K = x.shape
    N = B.shape[1]
    fusable = (x.dtype == torch.bfloat16 and B.dtype == torch.bfloat16 and M * K <= 32768 and K <= 8192 and K % 32 == 0
               and B.stride(0) == 1 and not torch.compiler.is_compiling() and ("norm_mm", M, N, K) not in _declined)
    if fusable:
        x2, ldx = _rows16(x)
        r2, ldr = (None, 0) if residual is None else _rows16(residual)
        w, ldb_k, ldb_n = _weight_operand(B)
        nw = None if norm_weight is None else norm_weight.contiguous()
        b = None if bias is None else bias.contiguous()
        C = torch.empty((M, N), device=x.device, dtype=x.dtype)
        rout = None if residual is None else torch.empty((M, K), device=x.device, dtype=x.dtype)
        rc = _lib.lib().bi_rmsnorm_gemm_bf16(x2.data_ptr(), ldx, None if r2 is None else r2.data_ptr(), ldr,
                                             None if nw is None else nw.data_ptr(), eps,
                                             None if rout is None else rout.data_ptr(), K, w.data_ptr(), ldb_k, ldb_n,
                                             C.data_ptr(), C.stride(0), M, N, K, None if b is None else b.data_ptr(), _stream(x))
        if rc == _lib.TBIK_OK:
            return C, rout
        if rc != _lib.TBIK_ERR_UNSUPPORTED:
            _lib.check(rc, "bi_rmsnorm_gemm_bf16")
        _declined.add(("norm_mm", M, N, K))
    if residual is None:
        h, rout = bi_rmsnorm(x, norm_weight, eps), None
    else:
        h, rout = bi_add_rmsnorm(x, residual, norm_weight, eps)
    return bi_gemm(h, B, bias), rout


def gemm_tree_silu_mul(gate: torch.Tensor, up: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor], leaf_k: int) -> torch.Tensor:
    """gemm_tree(silu(gate) * up, B, bias, leaf_k) for the two halves (or a K shard of both halves) of a merged gate/up
    projection: column slices of one tensor, same row stride.

    One launch (`tbik_gemm_silu_mul_bf16`) for a few bf16 rows, the activation kernel followed by the tree matmul
    otherwise.  Same bits either way."""
    _require_gpu(gate, up, B, bias)
    M, K = gate.shape
    N = B.shape[1]
    fusable = (gate.dtype == torch.bfloat16 and B.dtype == torch.bfloat16 and M <= 4 and up.shape == gate.shape
               and gate.stride(1) == 1 and up.stride(1) == 1 and gate.stride(0) == up.stride(0) and gate.stride(0) % 8 == 0
               and _aligned16(gate) and _aligned16(up) and B.stride(0) == 1 and not torch.compiler.is_compiling()
               and ("silu_tree", M, N, K, leaf_k) not in _declined)
    if fusable:
        w, ldb_k, ldb_n = _weight_operand(B)
        b = None if bias is None else bias.contiguous()
        C = torch.empty((M, N), device=gate.device, dtype=gate.dtype)
        rc = _lib.lib().tbik_gemm_silu_mul_bf16(gate.data_ptr(), up.data_ptr(), gate.stride(0) if M > 1 else max(gate.stride(0), K),
                                                w.data_ptr(), ldb_k, ldb_n, C.data_ptr(), C.stride(0), M, N, K, leaf_k,
                                                None if b is None else b.data_ptr(), _stream(gate))
        if rc == _lib.TBIK_OK:
            return C
        if rc != _lib.TBIK_ERR_UNSUPPORTED:
            _lib.check(rc, "tbik_gemm_silu_mul_bf16")
        _declined.add(("silu_tree", M, N, K, leaf_k))
    if (gate.dim() == 2 and up.shape == gate.shape and gate.stride(1) == 1 and up.stride(1) == 1 and gate.stride(0) == up.stride(0)
            and gate.dtype == up.dtype and up.data_ptr() == gate.data_ptr() + K * gate.element_size()
            and (M == 1 or gate.stride(0) >= 2 * K)):
        # the two halves of one merged projection, side by side in memory: the activation kernel reads them in place
        merged = torch.as_strided(gate, (M, 2 * K), (gate.stride(0), 1))
    else:
        merged = torch.cat((gate, up), dim=-1)
    return gemm_tree(bi_silu_mul(merged), B, bias, leaf_k)


def gemm_silu_mul(x: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
    """bi_silu_mul(bi_gemm(x, W.t())) for the merged gate/up weight W [2*inter, K] (nn.Linear layout): one launch
    (`bi_gemm_silu_mul_bf16`) for 5 .. 64 bf16 rows, the two calls otherwise.  Same bits either way."""
    _require_gpu(x, W)
    M, K = x.shape
    inter = W.shape[0] // 2
    fusable = (x.dtype == torch.bfloat16 and W.dtype == torch.bfloat16 and 4 < M <= 64 and W.shape[0] == 2 * inter and inter % 16 == 0
               and K % 32 == 0 and W.stride(1) == 1 and W.stride(0) % 8 == 0 and _aligned16(W) and not torch.compiler.is_compiling()
               and ("mm_silu", M, inter, K) not in _declined)
    if fusable:
        x2, ldx = _rows16(x)
        out = torch.empty((M, inter), device=x.device, dtype=x.dtype)
        rc = _lib.lib().bi_gemm_silu_mul_bf16(x2.data_ptr(), ldx, W.data_ptr(), W.stride(0), out.data_ptr(), out.stride(0), M, inter, K,
                                              _stream(x))
        if rc == _lib.TBIK_OK:
            return out
        if rc != _lib.TBIK_ERR_UNSUPPORTED:
            _lib.check(rc, "bi_gemm_silu_mul_bf16")
        _declined.add(("mm_silu", M, inter, K))
    return bi_silu_mul(bi_gemm(x, W.t(), None))


# --------------------------------------------------------------------------------------------
# the (add-)RMSNorm behind a row-split layer, inside the launch that combines the layer's K shards
# --------------------------------------------------------------------------------------------
def _norm_after(y: torch.Tensor, residual: Optional[torch.Tensor], norm_weight: Optional[torch.Tensor], eps: float):
    """The two-call form: (bi_rmsnorm(y [+ residual]), new residual or None)."""
    if residual is None:
        return bi_rmsnorm(y, norm_weight, eps), None
    out, res = bi_add_rmsnorm(y, residual, norm_weight, eps)
    return out, res


def gemm_tree_add_rmsnorm(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor], leaf_k: int,
                          residual: Optional[torch.Tensor], norm_weight: Optional[torch.Tensor], eps: float):
    """(rms_norm(gemm_tree(A, B, bias, leaf_k) [+ residual]) * norm_weight, new residual or None).

    One call (`tbik_gemm_rmsnorm_bf16`: the norm runs in the launch that combines the matmul's K shards) where the matmul
    of this shape ends in such a combine -- decode- and prefill-sized batches of a row-split layer; the matmul followed
    by the norm otherwise.  Same bits either way."""
    _require_gpu(A, B, bias, residual, norm_weight)
    M, K = A.shape
    N = B.shape[1]
    fusable = (A.dtype == torch.bfloat16 and B.dtype == torch.bfloat16 and M > 0 and N % 8 == 0 and N <= 8192 and B.stride(0) == 1
               and (residual is None or (residual.dtype == torch.bfloat16 and tuple(residual.shape) == (M, N)))
               and (norm_weight is None or norm_weight.dtype == torch.bfloat16) and (bias is None or bias.dtype == torch.bfloat16)
               and not torch.compiler.is_compiling() and ("tree_norm", M, N, K, leaf_k) not in _declined)
    if fusable:
        a, lda = _rows16(A)
        w, ldb_k, ldb_n = _weight_operand(B, M, True)
        if ldb_k == 1:
            L = _lib.lib()
            b = None if bias is None else bias.contiguous()
            nw = None if norm_weight is None else norm_weight.contiguous()
            r2, ldr = (None, 0) if residual is None else _rows16(residual)
            out = torch.empty((M, N), device=A.device, dtype=A.dtype)
            rout = None if residual is None else torch.empty_like(out)
            ws_bytes = L.tbik_gemm_workspace_bytes(M, N, K, leaf_k)
            ws = torch.empty(ws_bytes, device=A.device, dtype=torch.uint8) if ws_bytes else None
            rc = L.tbik_gemm_rmsnorm_bf16(a.data_ptr(), lda, w.data_ptr(), ldb_k, ldb_n, M, N, K, leaf_k,
                                          None if b is None else b.data_ptr(), None if r2 is None else r2.data_ptr(), ldr,
                                          None if nw is None else nw.data_ptr(), eps,
                                          None if rout is None else rout.data_ptr(), 0 if rout is None else rout.stride(0),
                                          out.data_ptr(), out.stride(0), None if ws is None else ws.data_ptr(), ws_bytes, _stream(A))
            if rc == _lib.TBIK_OK:
                return out, rout
            if rc != _lib.TBIK_ERR_UNSUPPORTED:
                _lib.check(rc, "tbik_gemm_rmsnorm_bf16")
            _declined.add(("tree_norm", M, N, K, leaf_k))
    return _norm_after(gemm_tree(A, B, bias, leaf_k), residual, norm_weight, eps)


def tree_combine_add_rmsnorm(parts: List[torch.Tensor], bias: Optional[torch.Tensor], residual: Optional[torch.Tensor],
                             norm_weight: Optional[torch.Tensor], eps: float):
    """(rms_norm(tree_combine(parts) (+ bias) [+ residual]) * norm_weight, new residual or None) for 2-D partials: one
    launch (`tbik_tree_combine_rmsnorm_bf16`) for bf16 rows of at most 8192 elements, the separate calls otherwise."""
    _require_gpu(*parts, bias, residual, norm_weight)
    p0 = parts[0]
    n = len(parts)
    fusable = (p0.dim() == 2 and n >= 2 and n <= 32 and (n & (n - 1)) == 0 and all(p.dtype == torch.bfloat16 and p.shape == p0.shape for p in parts)
               and p0.shape[0] > 0 and p0.shape[1] % 8 == 0 and p0.shape[1] <= 8192
               and (residual is None or (residual.dtype == torch.bfloat16 and residual.shape == p0.shape))
               and (norm_weight is None or norm_weight.dtype == torch.bfloat16) and (bias is None or bias.dtype == torch.bfloat16)
               and not torch.compiler.is_compiling())
    if fusable:
        ps = [p.contiguous() for p in parts]
        if all(_aligned16(p) for p in ps):
            M, N = p0.shape
            arr = (ctypes.c_void_p * n)(*[p.data_ptr() for p in ps])
            b = None if bias is None else bias.contiguous()
            nw = None if norm_weight is None else norm_weight.contiguous()
            r2, ldr = (None, 0) if residual is None else _rows16(residual)
            out = torch.empty((M, N), device=p0.device, dtype=p0.dtype)
            rout = None if residual is None else torch.empty_like(out)
            rc = _lib.lib().tbik_tree_combine_rmsnorm_bf16(arr, n, M, N, None if b is None else b.data_ptr(),
                                                           None if r2 is None else r2.data_ptr(), ldr,
                                                           None if nw is None else nw.data_ptr(), eps,
                                                           None if rout is None else rout.data_ptr(), 0 if rout is None else rout.stride(0),
                                                           out.data_ptr(), out.stride(0), _stream(p0))
            _lib.check(rc, "tbik_tree_combine_rmsnorm_bf16")
            return out, rout
    y = parts[0] if n == 1 else tree_combine(parts)
    if bias is not None:
        y = y + bias
    return _norm_after(y, residual, norm_weight, eps)


# --------------------------------------------------------------------------------------------
# q/k norm + rotary embedding + KV-cache write in front of the attention
# --------------------------------------------------------------------------------------------
def bi_qk_norm_rope_cache_bf16(qkv: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor, inv_freq: torch.Tensor,
                               positions: torch.Tensor, seq_of_token: torch.Tensor, k_cache: torch.Tensor,
                               vt_cache: torch.Tensor, q_heads: int, kv_heads: int, eps: float) -> torch.Tensor:
    """Writes this step's keys and values into the caches (in place) and returns the normed, rotated queries
    [tokens, q_heads, 128]."""
    _require_gpu(qkv, q_weight, k_weight, inv_freq, positions, seq_of_token, k_cache, vt_cache)
    tokens = qkv.shape[0]
    assert qkv.dtype == torch.bfloat16 and qkv.stride(1) == 1 and qkv.shape[1] == (q_heads + 2 * kv_heads) * 128
    assert k_cache.is_contiguous() and vt_cache.is_contiguous() and k_cache.shape[1] == kv_heads and k_cache.shape[3] == 128
    assert positions.dtype == torch.int64 and seq_of_token.dtype == torch.int64 and inv_freq.dtype == torch.float32
    assert positions.numel() == tokens and seq_of_token.numel() == tokens and inv_freq.numel() == 64
    q_out = torch.empty((tokens, q_heads, 128), device=qkv.device, dtype=torch.bfloat16)
    rc = _lib.lib().bi_qk_norm_rope_cache_bf16(
        qkv.data_ptr(), qkv.stride(0), q_weight.contiguous().data_ptr(), k_weight.contiguous().data_ptr(),
        inv_freq.contiguous().data_ptr(), positions.contiguous().data_ptr(), seq_of_token.contiguous().data_ptr(),
        q_out.data_ptr(), k_cache.data_ptr(), vt_cache.data_ptr(), tokens, q_heads, kv_heads, 128,
        k_cache.shape[2], k_cache.shape[0], eps, _stream(qkv))
    _lib.check(rc, "bi_qk_norm_rope_cache_bf16")
    return q_out


def bi_attention_decode_qkv(qkv: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor, inv_freq: torch.Tensor,
                            k_cache: torch.Tensor, vt_cache: torch.Tensor, ctx_len: torch.Tensor, q_heads: int, kv_heads: int,
                            scale: float, eps: float) -> torch.Tensor:
    """A decode step of an attention block for sequences with one new token each (row b of qkv = sequence b's token at
    position ctx_len[b] - 1): per-head q/k norm, rotary embedding, cache write (in place) and attention in one launch
    (`bi_attention_decode_qkv_bf16`), the two calls where that kernel does not apply.  Same bits either way."""
    _require_gpu(qkv, q_weight, k_weight, inv_freq, k_cache, vt_cache, ctx_len)
    B = qkv.shape[0]
    assert qkv.dtype == torch.bfloat16 and qkv.stride(1) == 1 and qkv.shape[1] == (q_heads + 2 * kv_heads) * 128
    assert k_cache.is_contiguous() and vt_cache.is_contiguous() and k_cache.shape[1] == kv_heads and k_cache.shape[3] == 128
    assert ctx_len.dtype == torch.int32 and ctx_len.numel() == B and k_cache.shape[0] == B and inv_freq.dtype == torch.float32
    max_len = k_cache.shape[2]
    if ("attn_qkv", q_heads, kv_heads, max_len % 32) not in _declined:
        out = torch.empty((B, q_heads, 128), device=qkv.device, dtype=qkv.dtype)
        rc = _lib.lib().bi_attention_decode_qkv_bf16(
            qkv.data_ptr(), qkv.stride(0) if B > 1 else max(qkv.stride(0), qkv.shape[1]), q_weight.contiguous().data_ptr(),
            k_weight.contiguous().data_ptr(), inv_freq.contiguous().data_ptr(), k_cache.data_ptr(), vt_cache.data_ptr(),
            out.data_ptr(), ctx_len.data_ptr(), B, q_heads, kv_heads, 128, max_len, scale, eps, _stream(qkv))
        if rc == _lib.TBIK_OK:
            return out
        if rc != _lib.TBIK_ERR_UNSUPPORTED:
            _lib.check(rc, "bi_attention_decode_qkv_bf16")
        _declined.add(("attn_qkv", q_heads, kv_heads, max_len % 32))
    pos = (ctx_len - 1).to(torch.int64)
    seq = torch.arange(B, device=qkv.device, dtype=torch.int64)
    q = bi_qk_norm_rope_cache_bf16(qkv, q_weight, k_weight, inv_freq, pos, seq, k_cache, vt_cache, q_heads, kv_heads, eps)
    one = torch.ones(B, dtype=torch.int32, device=qkv.device)
    return bi_attention_bf16(q, k_cache, vt_cache, torch.arange(B, dtype=torch.int32, device=qkv.device), one, ctx_len, 1, scale)


def bi_argmax(logits: torch.Tensor) -> torch.Tensor:
    """Index (int64) of the largest element of each row of a 2-D bf16 tensor, ties resolved to the lowest index."""
    _require_gpu(logits)
    if logits.dim() != 2 or logits.dtype != torch.bfloat16:
        raise NotImplementedError("bi_argmax takes a 2-D bfloat16 tensor")
    x = logits if logits.stride(1) == 1 else logits.contiguous()
    out = torch.empty((x.shape[0],), device=x.device, dtype=torch.int64)
    rc = _lib.lib().bi_argmax_bf16(x.data_ptr(), x.stride(0) if x.shape[0] > 1 else max(x.stride(0), x.shape[1]), out.data_ptr(), x.shape[0], x.shape[1], _stream(x))
    _lib.check(rc, "bi_argmax_bf16")
    return out


def bi_argmax_advance(logits: torch.Tensor, next_token: torch.Tensor, history: Optional[torch.Tensor] = None,
                      count: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
                      ctx_len: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bi_argmax written into `next_token` (int64 [rows]) plus the bookkeeping of a decode step in the same launch:
    the index also goes to history[r, count[r]] (int64 [rows, T]; skipped once count[r] reaches T), then count[r]
    (int64), positions[r] (int64) and ctx_len[r] (int32) advance by one.  All tensors are updated in place."""
    _require_gpu(logits)
    if logits.dim() != 2 or logits.dtype != torch.bfloat16:
        raise NotImplementedError("bi_argmax_advance takes a 2-D bfloat16 tensor")
    x = logits if logits.stride(1) == 1 else logits.contiguous()
    rows = x.shape[0]

    def arg(t, dtype, shape, name):
        if t is None:
            return 0
        if t.dtype != dtype or tuple(t.shape) != shape or not t.is_contiguous() or t.device != x.device:
            raise ValueError(f"{name}: a contiguous {dtype} tensor of shape {shape} on {x.device} is required")
        return t.data_ptr()

    if history is not None and (history.dim() != 2 or count is None):
        raise ValueError("history is [rows, T] and needs count")
    T = history.shape[1] if history is not None else 0
    rc = _lib.lib().bi_argmax_advance_bf16(
        x.data_ptr(), x.stride(0) if rows > 1 else max(x.stride(0), x.shape[1]),
        arg(next_token, torch.int64, (rows,), "next_token"), rows, x.shape[1],
        arg(history, torch.int64, (rows, T), "history"), T, arg(count, torch.int64, (rows,), "count"),
        arg(positions, torch.int64, (rows,), "positions"), arg(ctx_len, torch.int32, (rows,), "ctx_len"), _stream(x))
    _lib.check(rc, "bi_argmax_advance_bf16")
    return next_token
