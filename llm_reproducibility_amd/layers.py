"""Caller-side layers of the row-split path, shaped like the vLLM classes the reference patches.

`RowParallelLinear` carries the fields the reference's replacement forward reads
(src/patch/patch_tp_invariant.py:11-46): input_is_parallel, tp_rank, tp_size, reduce_results,
skip_bias_add, return_bias, quant_method, weight [N, K_shard], bias.  `SimulatedTPRowLinear` holds
all shards of one layer on one GPU and combines their outputs in the order the cross-GPU tree
all-reduce would use (simple_matmul.py:23-43 of the reference).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from .tbik.tree_based_matmul import choose_leaf_k, matmul_tp_persistent
from .tbik.tree_based_all_reduce import tree_all_reduce_sum, tree_combine
from .bio.batch_invariant_ops import rms_norm


class RowParallelLinear(nn.Module):
    """One rank's shard of a row-split linear layer (the input dimension is split across ranks)."""

    def __init__(self, input_size: int, output_size: int, bias: bool = False, tp_rank: int = 0, tp_size: int = 1,
                 input_is_parallel: bool = True, reduce_results: bool = True, skip_bias_add: bool = False,
                 return_bias: bool = False, tp_group=None, max_tp: int = 8, dtype=torch.bfloat16, device=None):
        super().__init__()
        assert input_size % tp_size == 0
        self.input_size = input_size
        self.output_size = output_size
        self.tp_rank, self.tp_size, self.tp_group = tp_rank, tp_size, tp_group
        self.input_is_parallel = input_is_parallel
        self.reduce_results = reduce_results
        self.skip_bias_add = skip_bias_add
        self.return_bias = return_bias
        self.quant_method = "unquantized"
        self.input_size_per_partition = input_size // tp_size
        # the leaf is a property of the LAYER (full K and the largest TP degree it may run at)
        self.tbik_leaf_k = choose_leaf_k(input_size, max(max_tp, tp_size))
        self.weight = nn.Parameter(torch.empty(output_size, self.input_size_per_partition, dtype=dtype, device=device),
                                   requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(output_size, dtype=dtype, device=device), requires_grad=False) if bias else None

    def forward(self, input_):
        """Stock behaviour (library GEMM + sum all-reduce); `patch_tp_invariant()` replaces it."""
        x = input_ if self.input_is_parallel else input_.chunk(self.tp_size, dim=-1)[self.tp_rank].contiguous()
        bias_ = None if (self.tp_rank > 0 or self.skip_bias_add) else self.bias
        out = torch.nn.functional.linear(x, self.weight, bias_)
        if self.reduce_results and self.tp_size > 1:
            torch.distributed.all_reduce(out, group=self.tp_group)
        out_bias = self.bias if self.skip_bias_add else None
        return (out, out_bias) if self.return_bias else out


def tbik_row_parallel_forward(self, input_):
    """TP-invariant forward of a row-split linear: tree matmul on the shard, tree all-reduce across ranks.

    Follows src/patch/patch_tp_invariant.py:11-46; the bias is added once, after the reduction, on every
    rank (the reference adds a rank-0-only alias there, which is None on the other ranks).
    """
    if self.input_is_parallel:
        input_parallel = input_
    else:
        input_parallel = input_.chunk(self.tp_size, dim=-1)[self.tp_rank].contiguous()
    assert self.quant_method is not None
    lead = input_parallel.shape[:-1]
    x2 = input_parallel.reshape(-1, input_parallel.shape[-1])
    leaf_k = getattr(self, "tbik_leaf_k", 256)
    output_parallel = matmul_tp_persistent(x2, self.weight.t(), leaf_k=leaf_k)
    if self.reduce_results and self.tp_size > 1:
        group = getattr(self, "tp_group", None)
        if group is None:
            try:  # vLLM keeps the group in its parallel state
                from vllm.distributed.parallel_state import get_tp_group
                group = get_tp_group().device_group
            except ImportError:
                group = None
        output = tree_all_reduce_sum(output_parallel, device_group=group)
    else:
        output = output_parallel
    if (not self.skip_bias_add) and self.bias is not None:
        # once per reduced output: on every rank after the tree all-reduce; on rank 0 only when the caller reduces
        # the partial outputs itself (reduce_results=False), or that reduction would add the bias tp_size times
        if self.reduce_results or self.tp_size == 1 or self.tp_rank == 0:
            output += self.bias
    output = output.reshape(*lead, output.shape[-1])
    output_bias = self.bias if self.skip_bias_add else None
    if not self.return_bias:
        return output
    return output, output_bias


class SimulatedTPRowLinear(nn.Module):
    """All `tp_size` shards of a row-split linear on ONE GPU: per-shard tree matmul, then the shard tree."""

    def __init__(self, weight: torch.Tensor, tp_size: int, bias: Optional[torch.Tensor] = None, max_tp: int = 8):
        super().__init__()
        N, K = weight.shape
        assert K % tp_size == 0
        self.tp_size = tp_size
        self.leaf_k = choose_leaf_k(K, max(max_tp, tp_size))
        self.weight = weight  # [N, K], K contiguous; shards are column slices (views)
        self.bias = bias

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        K = x2.shape[1]
        ks = K // self.tp_size
        parts = [matmul_tp_persistent(x2[:, r * ks:(r + 1) * ks], self.weight[:, r * ks:(r + 1) * ks].t(), leaf_k=self.leaf_k)
                 for r in range(self.tp_size)]
        out = parts[0] if self.tp_size == 1 else tree_combine(parts)
        if self.bias is not None:
            out = out + self.bias
        return out.reshape(*lead, out.shape[-1])

    def forward_add_norm(self, x: torch.Tensor, residual: Optional[torch.Tensor], norm_weight: Optional[torch.Tensor], eps: float):
        """(rms_norm(forward(x) [+ residual]) * norm_weight, new residual or None): the add-RMSNorm that follows a
        row-split layer in a decoder block, computed by the launch that combines the K shards where there is one
        (inside the matmul for one rank, the shard combine for several); same bits as forward() and the norm."""
        from . import ops
        x2 = x.reshape(-1, x.shape[-1])
        r2 = None if residual is None else residual.reshape(-1, residual.shape[-1])
        K = x2.shape[1]
        ks = K // self.tp_size
        if self.tp_size == 1:
            out, res = ops.gemm_tree_add_rmsnorm(x2, self.weight.t(), self.bias, self.leaf_k, r2, norm_weight, eps)
        else:
            parts = [matmul_tp_persistent(x2[:, r * ks:(r + 1) * ks], self.weight[:, r * ks:(r + 1) * ks].t(), leaf_k=self.leaf_k)
                     for r in range(self.tp_size)]
            out, res = ops.tree_combine_add_rmsnorm(parts, self.bias, r2, norm_weight, eps)
        lead = x.shape[:-1]
        out = out.reshape(*lead, out.shape[-1])
        return out, (None if res is None else res.reshape(*lead, res.shape[-1]))

    def forward_gated(self, gate_up: torch.Tensor) -> torch.Tensor:
        """forward(silu(gate) * up) for the merged projection gate_up = [gate | up]: the activation is formed inside the
        per-shard tree matmul where that is one launch (a few rows), by its own kernel otherwise; same bits."""
        from . import ops
        lead = gate_up.shape[:-1]
        g2 = gate_up.reshape(-1, gate_up.shape[-1])
        K = g2.shape[1] // 2
        assert K == self.weight.shape[1]
        if g2.shape[0] > 4 or g2.dtype != torch.bfloat16:
            return self.forward(ops.bi_silu_mul(g2)).reshape(*lead, self.weight.shape[0])
        ks = K // self.tp_size
        parts = [ops.gemm_tree_silu_mul(g2[:, r * ks:(r + 1) * ks], g2[:, K + r * ks:K + (r + 1) * ks],
                                        self.weight[:, r * ks:(r + 1) * ks].t(), None, self.leaf_k) for r in range(self.tp_size)]
        out = parts[0] if self.tp_size == 1 else tree_combine(parts)
        if self.bias is not None:
            out = out + self.bias
        return out.reshape(*lead, out.shape[-1])


class RMSNorm(nn.Module):
    """RMSNorm with vLLM's call shape: forward(x, residual=None) -> out | (out, new_residual)."""

    def __init__(self, hidden_size: int, eps: float = 1e-6, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device), requires_grad=False)
        self.variance_epsilon = eps

    def forward_native(self, x, residual=None):
        orig = x.dtype
        x = x.float()
        if residual is not None:
            x = x + residual.float()
            residual = x.to(orig)
        var = x.pow(2).mean(dim=-1, keepdim=True)
        x = (x * torch.rsqrt(var + self.variance_epsilon)).to(orig) * self.weight
        return x if residual is None else (x, residual)

    def forward_fused(self, x, residual=None):
        if x.dtype not in (torch.bfloat16, torch.float16) or x.shape[-1] > 8192 or x.shape[-1] % 8 != 0:
            return self.forward_native(x, residual)   # shapes and dtypes the fused kernel does not take
        return rms_norm(x, self.weight, self.variance_epsilon, residual)

    forward = forward_native
