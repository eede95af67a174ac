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


def _fake_world(monkeypatch, partials):
    import torch.distributed as dist
    monkeypatch.setattr(dist, "get_world_size", lambda group=None: len(partials))

    def fake_all_gather(out_list, inp, group=None):
        assert len(out_list) == len(partials) and inp.is_cuda and inp.is_contiguous()
        for o, part in zip(out_list, partials):
            o.copy_(part)
    monkeypatch.setattr(dist, "all_gather", fake_all_gather)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_tree_all_reduce_sum_over_a_gathered_world(dev, monkeypatch, dtype):
    """The wrapper the patched layer calls, with the gather replaced by a stand-in that delivers the other ranks'
    partials (one GPU here): the HIP combine must give the CPU oracle's adjacent-pair tree bit for bit, for worlds of
    1/2/4/8, in bf16, fp16 and fp32 (an fp32 node is one fp32 addition: only the order has to match)."""
    from llm_reproducibility_amd.tbik.tree_based_all_reduce import tree_all_reduce_sum, tree_all_reduce_sum_native
    shape = (37, 24)                       # 888 elements: vector body + scalar tail in the fp32 kernel (numel % 4 == 0)
    for n in (1, 2, 4, 8):
        cpu = [(torch.randn(shape, generator=torch.Generator().manual_seed(100 + r)) * 50).to(dtype) for r in range(n)]
        _fake_world(monkeypatch, [p.to(dev) for p in cpu])
        want = O.tree_combine(cpu)
        x = cpu[0].to(dev)
        for fn in (tree_all_reduce_sum, tree_all_reduce_sum_native):
            got = fn(x)
            assert got.dtype == dtype and got.data_ptr() != x.data_ptr()
            assert torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8)), (n, dtype)
    _fake_world(monkeypatch, [torch.zeros(shape, dtype=dtype, device=dev)] * 3)
    with pytest.raises(ValueError):
        tree_all_reduce_sum(torch.zeros(shape, dtype=dtype, device=dev))


def test_fp32_tree_combine_kernel_on_ragged_and_misaligned_buffers(dev):
    from llm_reproducibility_amd.tbik import tree_combine
    g = torch.Generator().manual_seed(3)
    for n in (1, 2, 4, 8, 16, 32):
        for numel in (1, 3, 4, 1023, 4096 + 5):
            cpu = [torch.randn(numel + 1, generator=g) * 1e3 for _ in range(n)]
            want = O.tree_combine([c[1:] for c in cpu])
            got = tree_combine([c.to(dev)[1:] for c in cpu])        # 4-byte aligned views: the scalar path
            assert torch.equal(got.cpu(), want), (n, numel)
            got = tree_combine([c[1:].to(dev) for c in cpu])        # fresh (aligned) buffers: the vector path
            assert torch.equal(got.cpu(), want), (n, numel)


def test_row_parallel_forward_reduces_through_the_tree_and_adds_the_bias_once(dev, monkeypatch):
    """tbik_row_parallel_forward on rank r of a world of 4 (the other ranks' partial outputs come from a stand-in for
    the gather): output == oracle tree over the four shard products + bias; with reduce_results=False the bias is added
    on rank 0 only, so that an external reduction adds it once."""
    K, N, tp = 4096, 64, 4
    W = O.integer_bf16((N, K), -7, 7, 0)
    bias = O.integer_bf16((N,), -100, 100, 1)
    x = O.integer_bf16((5, K), -9, 9, 2)
    ks = K // tp
    shard_out = [O.matmul_tree(x[:, r * ks:(r + 1) * ks], W[:, r * ks:(r + 1) * ks].t()) for r in range(tp)]
    want = O.tree_combine(shard_out) + bias
    assert torch.equal(O.tree_combine(shard_out), O.matmul_tree(x, W.t()))       # shard tree o leaf tree = full tree
    _fake_world(monkeypatch, [s.to(dev) for s in shard_out])
    for rank in (0, 2):
        layer = layers.RowParallelLinear(K, N, bias=True, tp_rank=rank, tp_size=tp, device=dev)
        layer.weight.copy_(W[:, rank * ks:(rank + 1) * ks].to(dev))
        layer.bias.copy_(bias.to(dev))
        got = layers.tbik_row_parallel_forward(layer, x[:, rank * ks:(rank + 1) * ks].to(dev))
        assert torch.equal(got.cpu(), want), rank
        layer.reduce_results = False
        part = layers.tbik_row_parallel_forward(layer, x[:, rank * ks:(rank + 1) * ks].to(dev))
        assert torch.equal(part.cpu(), shard_out[rank] + bias if rank == 0 else shard_out[rank]), rank
        layer.input_is_parallel = False                                              # the layer splits the input itself
        part2 = layers.tbik_row_parallel_forward(layer, x.to(dev))
        assert torch.equal(part2, part), rank


def test_tree_all_reduce_sum_in_a_real_process_group_of_one(dev):
    """The wrapper through torch.distributed itself: a world of size 1 on the RCCL backend (this box has one GPU).  The
    gather then returns the rank's own partial and the tree over one partial is the identity, in a new tensor."""
    import datetime
    import socket
    import torch.distributed as dist
    from llm_reproducibility_amd.tbik.tree_based_all_reduce import tree_all_reduce_sum
    if dist.is_initialized():
        pytest.skip("a process group already exists in this process")
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    print("case process group of one, port", port, flush=True)
    dist.init_process_group("nccl", init_method=f"tcp://127.0.0.1:{port}", rank=0, world_size=1,
                            timeout=datetime.timedelta(seconds=60), device_id=dev)
    try:
        x = O.gaussian_bf16((33, 512), 1.0, 0).to(dev)
        got = tree_all_reduce_sum(x)
        torch.cuda.synchronize()
        assert torch.equal(got, x) and got.data_ptr() != x.data_ptr()
        got2 = tree_all_reduce_sum(x, device_group=dist.group.WORLD)
        assert torch.equal(got2, x)
    finally:
        dist.destroy_process_group()
