"""Invariance check of one matmul, selected by TP_INVARIANT_MATMUL.

    TP_INVARIANT_MATMUL=1 python -m llm_reproducibility_amd.check_matmul [--m 1024 --k 6144 --n 2048 --shards 4]

With the flag on, the product is `matmul_tp_persistent` (tree-ordered, this library's HIP kernels); with it off (the
default), `torch.matmul` of the vendor library.  Two differences are printed and returned, as the reference's smoke
script reports them (simple_matmul.py:8-43; this file shares only its purpose and its switch):

  batch   rows [0, M/2) of f(A, B) against f(A[:M/2], B): the same rows computed in a batch of another size
  shards  f(A, B) against the K axis cut into `shards` contiguous slices, one product each, the partial results
          added pairwise in a binary tree in the operands' dtype (any power of two, not only four)

Both are exactly 0.0 for the tree-ordered matmul; the library matmul usually fails the second and, depending on the
shape, the first.  `run()` returns the two numbers so that tests can assert on them; the exit status is 0 when the
selected product is invariant, 1 otherwise.
"""
from __future__ import annotations

import argparse
import sys

import torch

from . import utils


def select_matmul():
    """The product under test: the tree-ordered kernel when TP_INVARIANT_MATMUL is set, else torch.matmul."""
    if utils.tp_invariant_matmul_is_enabled():
        from .tbik import matmul_tp_persistent
        return matmul_tp_persistent, "matmul_tp_persistent"
    return torch.matmul, "torch.matmul"


def pairwise_tree_sum(parts):
    """((p0 + p1) + (p2 + p3)) + ...: adjacent pairs first, every add rounded to the parts' dtype."""
    parts = list(parts)
    if len(parts) & (len(parts) - 1):
        raise ValueError("the number of shards must be a power of two")
    while len(parts) > 1:
        parts = [parts[i] + parts[i + 1] for i in range(0, len(parts), 2)]
    return parts[0]


def run(m: int = 1024, k: int = 6144, n: int = 2048, shards: int = 4, seed: int = 0, device: str = "cuda:0",
        dtype: torch.dtype = torch.bfloat16):
    f, name = select_matmul()
    g = torch.Generator().manual_seed(seed)
    a = torch.randn((m, k), generator=g).to(dtype).to(device)
    b = torch.randn((k, n), generator=g).to(dtype).to(device)
    full = f(a, b)
    batch_diff = (full[: m // 2].float() - f(a[: m // 2], b).float()).abs().max().item()
    if k % shards:
        raise ValueError(f"K={k} is not a whole number of {shards} shards")
    ks = k // shards
    parts = [f(a[:, r * ks:(r + 1) * ks], b[r * ks:(r + 1) * ks, :]) for r in range(shards)]
    shard_diff = (full.float() - pairwise_tree_sum(parts).float()).abs().max().item()
    return name, batch_diff, shard_diff


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--m", type=int, default=1024)
    ap.add_argument("--k", type=int, default=6144)
    ap.add_argument("--n", type=int, default=2048)
    ap.add_argument("--shards", type=int, default=4)
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args(argv)
    name, batch_diff, shard_diff = run(args.m, args.k, args.n, args.shards, args.seed)
    print(f"product: {name}  (TP_INVARIANT_MATMUL={int(utils.tp_invariant_matmul_is_enabled())})")
    print(f"batch  invariance, M={args.m} against M={args.m // 2}: max |diff| = {batch_diff}")
    print(f"shard  invariance, K={args.k} in {args.shards} shards + pairwise tree: max |diff| = {shard_diff}")
    return 0 if batch_diff == 0.0 and shard_diff == 0.0 else 1


if __name__ == "__main__":
    sys.exit(main())
