"""Tree all-reduce of row-split partial outputs.

Drop-in for the reference's src/tbik/tree_based_all_reduce.py: every rank gathers all partials and
adds them in the fixed adjacent-pair tree, in the tensor's dtype.  The adds run in one HIP kernel
(csrc/tree_combine.hip) instead of world_size-1 elementwise launches.  `tree_combine` is the same
arithmetic on partials that already sit on one GPU (simulated tensor parallelism,
simple_matmul.py:35-38 of the reference).
"""
from __future__ import annotations

from typing import Sequence

import torch
import torch.distributed as dist

from .. import ops


def tree_combine(parts: Sequence[torch.Tensor]) -> torch.Tensor:
    """Adjacent-pair binary tree over a power-of-two number of same-shaped partials; returns a new tensor."""
    n = len(parts)
    if n == 0 or n & (n - 1) != 0:
        raise ValueError("the number of partials must be a power of 2")
    if n > 32:
        # wider worlds: reduce groups of 32 first; adjacent-pair trees compose
        return tree_combine([tree_combine(parts[i:i + 32]) for i in range(0, n, 32)])
    if any(p.dtype != parts[0].dtype for p in parts):
        raise NotImplementedError("tree_combine takes partials of one dtype")
    if any(p.shape != parts[0].shape for p in parts):
        raise ValueError("partials must have the same shape")
    if parts[0].dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError("tree_combine is implemented for bfloat16, float16 and float32 partials")
    return ops.tree_combine(list(parts))


def tree_all_reduce_sum_native(x: torch.Tensor, device_group=None) -> torch.Tensor:
    world_size = dist.get_world_size(device_group)
    if world_size & (world_size - 1) != 0:
        raise ValueError("world_size must be a power of 2 to use the tree all-reduce")
    result = [torch.empty_like(x) for _ in range(world_size)]
    dist.all_gather(result, x.contiguous(), group=device_group)
    return tree_combine(result)


def tree_all_reduce_sum(x: torch.Tensor, device_group=None) -> torch.Tensor:
    """Same result on every rank, bitwise equal to the single-GPU tree over the same partials."""
    return tree_all_reduce_sum_native(x, device_group)
