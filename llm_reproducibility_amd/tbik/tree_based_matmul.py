"""TP-invariant (tree-ordered) matmul for row-split layers: host wrapper over the gfx950 MFMA kernel.

Drop-in for the reference's `matmul_tp_persistent` (src/tbik/tree_based_matmul.py:190-277): same
signature, same assertions, output allocated here, inputs never modified.  The arithmetic contract
(leaf = fp32 MFMA chain over `leaf_k` consecutive k rounded to bf16; level 0 left-to-right over FLB
leaves; adjacent-pair binary tree above; every node bf16) is implemented in csrc/gemm_tiled.hip.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops

LEAF_K_DEFAULT = 256  # BLOCK_SIZE_K of the reference's bf16 config, src/tbik/tree_based_matmul.py:206-214


def choose_leaf_k(global_k: int, max_tp: int = 8) -> int:
    """Leaf size for a row-split layer whose FULL reduction extent is `global_k`.

    The leaf has to be a property of the layer, not of a shard: every TP degree up to `max_tp` must
    cut its shard into whole leaves of the same size or the shards would build different trees.  256
    (the reference's value) is kept whenever global_k / max_tp is a multiple of 256; 128 otherwise
    (Qwen3-32B down_proj: 25600 / 8 = 3200 = 25 * 128).
    """
    for leaf in (256, 128):
        if global_k % (max_tp * leaf) == 0:
            return leaf
    raise ValueError(f"K={global_k} cannot be cut into whole leaves of 256 or 128 at TP={max_tp}")


def matmul_tp_persistent(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor] = None,
                         leaf_k: int = LEAF_K_DEFAULT) -> torch.Tensor:
    """C[M,N] = tree-ordered A[M,K] @ B[K,N] (+ bias), bf16, bitwise independent of M and of how K was sharded.

    A may be a column slice of a wider tensor (row stride > K); B is used in place when it is the
    transposed view of an nn.Linear weight ([N,K], K contiguous) and repacked once otherwise.
    """
    assert A.shape[-1] == B.shape[-2], "Dim doesn't match"
    assert A.dim() == 2 and B.dim() == 2, "2-D operands only"
    if A.dtype != B.dtype or A.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError("the gfx950 tree matmul takes bfloat16, float16 or float32 operands of one dtype")
    if A.dtype == torch.float32 and leaf_k == LEAF_K_DEFAULT:
        leaf_k = 128  # the reference's float32 configuration cuts K into leaves of 128 (:223-231)
    K = A.shape[1]
    assert K % leaf_k == 0, f"K={K} must be a multiple of the leaf size {leaf_k}"
    if bias is not None:
        assert bias.dim() == 1 and bias.shape[0] == B.shape[1] and bias.dtype == A.dtype
    return ops.gemm_tree(A, B, bias, leaf_k)
