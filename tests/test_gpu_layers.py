"""Caller side of the row-split path on the GPU: patched RowParallelLinear, simulated TP, fused RMSNorm module."""
import pytest
import torch

from oracle import tbik_oracle as O
from llm_reproducibility_amd import layers
from llm_reproducibility_amd.patch import patch_tp_invariant as ptp_fn
import importlib

pytestmark = pytest.mark.gpu


def test_simulated_tp_row_linear_is_tp_and_batch_invariant(dev):
    K, N = 12288, 4096
    W = O.gaussian_bf16((N, K), 0.02, 1).to(dev)
    x = O.silu_gated_bf16((2, 65, K), 0).to(dev)            # [batch, tokens, K]
    outs = [layers.SimulatedTPRowLinear(W, p)(x) for p in (1, 2, 4, 8)]
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    assert outs[0].shape == (2, 65, N)
    one = layers.SimulatedTPRowLinear(W, 4)(x[1:2, 7:8])
    assert torch.equal(one, outs[0][1:2, 7:8])
    want = O.matmul_tree(x[0, :8].cpu(), W.cpu().t())
    assert O.bf16_ulp_distance(outs[0][0, :8].cpu(), want).max() <= 1 or \
        (outs[0][0, :8].cpu().float() - want.float()).abs().max() <= 2 ** -8 * want.float().abs().max()


def test_patched_row_parallel_linear_matches_tree_matmul(dev):
    ptp = importlib.import_module("llm_reproducibility_amd.patch.patch_tp_invariant")
    layer = layers.RowParallelLinear(1536, 128, bias=True, tp_rank=0, tp_size=1, max_tp=2, device=dev)
    layer.weight.copy_(O.integer_bf16((128, 1536), -7, 7, 0).to(dev))
    layer.bias.copy_(O.integer_bf16((128,), -100, 100, 1).to(dev))
    x = O.integer_bf16((3, 5, 1536), -9, 9, 2).to(dev)
    ptp_fn()
    try:
        got = layer(x)
    finally:
        ptp.unpatch_row_linear()
    want = O.matmul_tree(x.cpu().reshape(15, 1536), layer.weight.cpu().t(), layer.bias.cpu()).reshape(3, 5, 128)
    assert torch.equal(got.cpu(), want)
    stock = layer(x)                                   # library GEMM: close, not necessarily equal
    assert (stock.float() - got.float()).abs().max() <= 2 ** -6 * got.float().abs().max()


def test_rmsnorm_module_fused_vs_native(dev):
    m = layers.RMSNorm(4096, device=dev)
    m.weight.copy_(O.gaussian_bf16((4096,), 1.0, 0).to(dev))
    x = O.gaussian_bf16((33, 4096), 1.0, 1).to(dev)
    r = O.gaussian_bf16((33, 4096), 1.0, 2).to(dev)
    a = m.forward_native(x)
    b = m.forward_fused(x)
    assert O.bf16_ulp_distance(a.cpu(), b.cpu()).max() <= 2
    a2, ra = m.forward_native(x, r)
    b2, rb = m.forward_fused(x, r)
    assert torch.equal(ra, rb) and O.bf16_ulp_distance(a2.cpu(), b2.cpu()).max() <= 2
