"""Batch-invariant operator overrides backed by the gfx950 kernels.

Mirrors the public surface of the reference's src/bio/batch_invariant_ops.py: the same four mode
functions, the same five aten overrides on the GPU dispatch key ("CUDA" is the key ROCm tensors
use), the same helper names.  Each override's per-row result is independent of how many rows are in
the call because the kernels fix the reduction order as a function of the row length only.
"""
from __future__ import annotations

import contextlib
from collections import namedtuple
from typing import Optional

import torch

from .. import ops

__all__ = ["set_batch_invariant_mode", "is_batch_invariant_mode_enabled", "disable_batch_invariant_mode",
           "enable_batch_invariant_mode"]


# ---------------------------------------------------------------------------------------------
# operators
# ---------------------------------------------------------------------------------------------
def matmul_persistent(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a[M,K] @ b[K,N] (+ bias[N]) with one fp32 accumulator run sequentially over K (reference :127-197).

    Unlike the reference, the fp32 accumulator is rounded ONCE to the output dtype (the reference's
    kernel rounds through fp16 first, :119-123).
    """
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert a.dtype == b.dtype, "Incompatible dtypes"
    assert bias is None or bias.dim() == 1, "Currently assuming bias is 1D"
    if a.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError(f"batch-invariant mm on gfx950 takes bfloat16, float16 or float32, got {a.dtype}")
    if bias is not None and bias.dtype != a.dtype:
        bias = bias.to(a.dtype)
    return ops.bi_gemm(a, b, bias)


def log_softmax(input: torch.Tensor, dim: int = -1) -> torch.Tensor:
    """log_softmax over the last dimension (reference :263-301); output dtype = input dtype."""
    if dim != -1 and dim != input.ndim - 1:
        raise ValueError("This implementation only supports log_softmax along the last dimension")
    return _run_softmax(input, False, False)


def softmax(input: torch.Tensor, dim: int = -1) -> torch.Tensor:
    if dim != -1 and dim != input.ndim - 1:
        raise ValueError("This implementation only supports softmax along the last dimension")
    return _run_softmax(input, True, False)


def mean_dim(input: torch.Tensor, dim: int, keepdim: bool = False, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Mean over one dimension with a fixed accumulation order (reference :352-439)."""
    assert input.is_cuda, "Input must be a GPU tensor"
    assert -input.ndim <= dim < input.ndim, f"Invalid dimension {dim} for tensor with {input.ndim} dimensions"
    if dtype is None:
        dtype = torch.float32 if input.dtype in (torch.int8, torch.int16, torch.int32, torch.int64) else input.dtype
    if input.dtype != dtype:
        input = input.to(dtype)
    return ops.bi_mean_dim(input, dim, keepdim)


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, residual: Optional[torch.Tensor] = None):
    """Fused RMSNorm (optionally add-residual first) with the arithmetic of vLLM's forward_native, which is
    what the reference routes RMSNorm to (src/patch/patch_batch_invariant.py:9-16).  Returns `out`, or
    `(out, new_residual)` when a residual is given."""
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError("rms_norm on gfx950 is implemented for bfloat16 and float16")
    if residual is None:
        return ops.bi_rmsnorm(x, weight, eps)
    out, new_res = ops.bi_add_rmsnorm(x, residual, weight, eps)
    return out, new_res


# ---------------------------------------------------------------------------------------------
# aten overrides (reference :442-472)
# ---------------------------------------------------------------------------------------------
def mm_batch_invariant(a, b):
    return matmul_persistent(a, b)


def addmm_batch_invariant(bias, a, b):
    return matmul_persistent(a, b, bias=bias)


def _run_softmax(input, write_softmax: bool, to_float: bool):
    """fp32, bf16 and fp16 go to the kernel as they are (it reads the input dtype itself); anything else is computed
    in fp32 and cast back."""
    if input.dtype in (torch.float32, torch.bfloat16, torch.float16):
        return ops.bi_log_softmax(input, write_softmax, to_float)
    out = ops.bi_log_softmax(input.float(), write_softmax, False)
    return out if to_float else out.to(input.dtype)


def _log_softmax_batch_invariant(input, dim, _half_to_float):
    if dim != -1 and dim != input.ndim - 1:
        raise ValueError("This implementation only supports softmax along the last dimension")
    return _run_softmax(input, False, bool(_half_to_float))


def _softmax_batch_invariant(input, dim, _half_to_float):
    if dim != -1 and dim != input.ndim - 1:
        raise ValueError("This implementation only supports softmax along the last dimension")
    return _run_softmax(input, True, bool(_half_to_float))


def mean_batch_invariant(input, dim, keepdim=False, dtype: Optional[torch.dtype] = None):
    assert dtype is None or dtype == torch.float32, f"unsupported dtype: {dtype}"
    if len(dim) == 1:
        return mean_dim(input, dim[0], keepdim=keepdim)
    assert input.dtype in {torch.float16, torch.bfloat16, torch.float32}, "only float types supported for now"
    if len(dim) == 0:
        dim = list(range(input.ndim))
    # several dims: fold them one at a time, innermost first; each fold is a fixed-order mean and the
    # product of the per-dim divisors is the element count
    out = input.float()
    for d in sorted((d % input.ndim for d in dim), reverse=True):
        out = ops.bi_mean_dim(out, d, True)
    if not keepdim:
        for d in sorted((d % input.ndim for d in dim), reverse=True):
            out = out.squeeze(d)
    return out.to(dtype or input.dtype)


# ---------------------------------------------------------------------------------------------
# mode switches (reference :475-516)
# ---------------------------------------------------------------------------------------------
_batch_invariant_MODE = False
_batch_invariant_LIB = None


def is_batch_invariant_mode_enabled():
    return _batch_invariant_MODE


def enable_batch_invariant_mode():
    global _batch_invariant_MODE, _batch_invariant_LIB
    if _batch_invariant_MODE:
        return
    _batch_invariant_MODE = True
    _batch_invariant_LIB = torch.library.Library("aten", "IMPL")
    _batch_invariant_LIB.impl("aten::mm", mm_batch_invariant, "CUDA")
    _batch_invariant_LIB.impl("aten::addmm", addmm_batch_invariant, "CUDA")
    _batch_invariant_LIB.impl("aten::_log_softmax", _log_softmax_batch_invariant, "CUDA")
    _batch_invariant_LIB.impl("aten::mean.dim", mean_batch_invariant, "CUDA")
    _batch_invariant_LIB.impl("aten::_softmax", _softmax_batch_invariant, "CUDA")


def disable_batch_invariant_mode():
    global _batch_invariant_MODE, _batch_invariant_LIB
    if _batch_invariant_LIB is not None:
        _batch_invariant_LIB._destroy()
    _batch_invariant_MODE = False
    _batch_invariant_LIB = None


@contextlib.contextmanager
def set_batch_invariant_mode(enabled: bool = True):
    global _batch_invariant_MODE, _batch_invariant_LIB
    old_mode = _batch_invariant_MODE
    if enabled:
        enable_batch_invariant_mode()
    else:
        disable_batch_invariant_mode()
    try:
        yield
    finally:
        # restore by re-registering: a destroyed Library object cannot be revived
        if old_mode:
            enable_batch_invariant_mode()
        else:
            disable_batch_invariant_mode()


AttentionBlockSize = namedtuple("AttentionBlockSize", ["block_m", "block_n"])


def get_batch_invariant_attention_block_size() -> AttentionBlockSize:
    return AttentionBlockSize(block_m=16, block_n=16)
