"""One-launch compositions for decode-sized batches against the two-launch forms they stand for (bit for bit) and
against the CPU oracle: RMSNorm inside the batch-invariant mm (`bi_rmsnorm_gemm_bf16`), SiLU * up inside the tree
matmul of down_proj (`tbik_gemm_silu_mul_bf16`)."""
import pytest
import torch

from oracle import tbik_oracle as O
from llm_reproducibility_amd import _lib, ops
from llm_reproducibility_amd.bio import batch_invariant_ops as bio
from llm_reproducibility_amd.decoder import DecoderConfig, Qwen3Decoder
from llm_reproducibility_amd.layers import SimulatedTPRowLinear
from llm_reproducibility_amd.tbik import matmul_tp_persistent

pytestmark = pytest.mark.gpu


def _raw_rmsnorm_gemm(x, res, w, eps, W, C, rout):
    s = torch.cuda.current_stream().cuda_stream
    M, K = x.shape
    return _lib.lib().bi_rmsnorm_gemm_bf16(x.data_ptr(), x.stride(0), None if res is None else res.data_ptr(), K,
                                           w.data_ptr(), eps, None if rout is None else rout.data_ptr(), K, W.data_ptr(), 1,
                                           W.stride(0), C.data_ptr(), C.stride(0), M, W.shape[0], K, None, s)


@pytest.mark.parametrize("M,K,N", [(1, 4096, 6144), (3, 4096, 24576), (4, 4096, 3000), (2, 8192, 5120), (1, 8192, 1024),
                                   (16, 1024, 4096), (7, 2048, 2048), (1, 4096, 151936)])
def test_rmsnorm_inside_the_mm_equals_the_two_launches(dev, M, K, N):
    x = O.gaussian_bf16((M, K), 1.0, 10 + M).to(dev)
    res = O.gaussian_bf16((M, K), 1.0, 20 + M).to(dev)
    w = (1.0 + 0.1 * torch.randn(K, generator=torch.Generator().manual_seed(3))).to(torch.bfloat16).to(dev)
    W = O.gaussian_bf16((N, K), 0.02, 30).to(dev)
    print("case rmsnorm+mm", M, K, N, flush=True)
    # the raw entry point takes the shape (so the wrapper below did not fall back to the two launches)
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    rout = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    assert _raw_rmsnorm_gemm(x, res, w, 1e-6, W, C, rout) == _lib.TBIK_OK
    h, new_res = bio.rms_norm(x, w, 1e-6, residual=res)
    want = bio.matmul_persistent(h, W.t())
    assert torch.equal(C, want) and torch.equal(rout, new_res)
    got, got_res = ops.rmsnorm_gemm(x, w, 1e-6, res, W.t())
    assert torch.equal(got, want) and torch.equal(got_res, new_res)
    # without a residual, and with a bias on the product
    bias = O.gaussian_bf16((N,), 1.0, 40).to(dev)
    got2, none = ops.rmsnorm_gemm(x, w, 1e-6, None, W.t(), bias)
    assert none is None and torch.equal(got2, bio.matmul_persistent(bio.rms_norm(x, w, 1e-6), W.t(), bias=bias))
    # against the CPU oracle of the composition (stated tolerance of the matmul: 1 ulp or 2^-8 of the scale)
    if N <= 24576:
        oh, ores = O.rmsnorm(x.cpu(), w.cpu(), 1e-6, residual=res.cpu())
        assert torch.equal(got_res.cpu(), ores)
        assert not O.outside_tolerance(got, O.matmul_single_acc(oh, W.cpu().t())).any()
    # a row alone equals the row in the batch
    one, _ = ops.rmsnorm_gemm(x[M - 1:], w, 1e-6, res[M - 1:], W.t())
    assert torch.equal(one[0], got[M - 1])


def test_rmsnorm_inside_the_mm_declines_what_it_cannot_stage(dev):
    K, N = 4096, 6144
    w = torch.ones(K, dtype=torch.bfloat16, device=dev)
    W = O.gaussian_bf16((N, K), 0.02, 1).to(dev)
    for M in (5, 64, 300):
        x = O.gaussian_bf16((M, K), 1.0, M).to(dev)
        C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        assert _raw_rmsnorm_gemm(x, None, w, 1e-6, W, C, None) == _lib.TBIK_ERR_UNSUPPORTED
        got, _ = ops.rmsnorm_gemm(x, w, 1e-6, None, W.t())        # the wrapper runs the two launches
        assert torch.equal(got, bio.matmul_persistent(bio.rms_norm(x, w, 1e-6), W.t()))
    # the new residual must not overwrite what other work-groups still read
    x = O.gaussian_bf16((1, K), 1.0, 0).to(dev)
    C = torch.empty((1, N), dtype=torch.bfloat16, device=dev)
    assert _raw_rmsnorm_gemm(x, x.clone(), w, 1e-6, W, C, x) == _lib.TBIK_ERR_INVALID


@pytest.mark.parametrize("M,K,N,leaf", [(1, 12288, 4096, 256), (3, 12288, 4096, 256), (2, 1536, 4096, 256), (3, 6144, 4096, 256),
                                        (1, 4096, 4096, 256), (2, 3072, 2048, 128), (4, 8192, 4096, 256)])
def test_silu_mul_inside_the_tree_matmul_equals_the_two_launches(dev, M, K, N, leaf):
    gu = (torch.randn((M, 2 * K), generator=torch.Generator().manual_seed(M + K)) * 2).to(torch.bfloat16).to(dev)
    W = O.gaussian_bf16((N, K), 0.02, 5).to(dev)
    print("case silu_mul+tree matmul", M, K, N, leaf, flush=True)
    s = torch.cuda.current_stream().cuda_stream
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    rc = _lib.lib().tbik_gemm_silu_mul_bf16(gu.data_ptr(), gu.data_ptr() + 2 * K, 2 * K, W.data_ptr(), 1, K, C.data_ptr(), N,
                                            M, N, K, leaf, None, s)
    assert rc == _lib.TBIK_OK
    act = ops.bi_silu_mul(gu)
    want = matmul_tp_persistent(act, W.t(), leaf_k=leaf)
    assert torch.equal(C, want)
    bias = O.gaussian_bf16((N,), 1.0, 6).to(dev)
    got = ops.gemm_tree_silu_mul(gu[:, :K], gu[:, K:], W.t(), bias, leaf)
    assert torch.equal(got, matmul_tp_persistent(act, W.t(), bias, leaf_k=leaf))
    # the CPU oracles of the two steps, each at its own tolerance: the activation within one rounding step of the
    # oracle's (device and host exponentials differ in the last bits), the product of THAT activation within the
    # tolerance of the tree matmul (a one-step change of an input can move a bf16 node of the tree by one of ITS
    # steps, which a cancelling output then shows at full size: the composition has no tighter bound than its parts)
    assert O.bf16_ulp_distance(act.cpu(), O.silu_mul(gu.cpu())).max() <= 1
    assert not O.outside_tolerance(C, O.matmul_tree(act.cpu(), W.cpu().t(), leaf=leaf)).any()
    assert torch.equal(ops.gemm_tree_silu_mul(gu[:1, :K], gu[:1, K:], W.t(), None, leaf)[0], C[0])


def test_silu_mul_inside_the_tree_matmul_over_simulated_shards(dev):
    """down_proj of the 8B configuration cut into 1/2/4/8 K shards, activation formed inside each shard's matmul:
    bitwise equal to the unsharded product of the stand-alone activation, and to the same layer without fusion."""
    K, N = 12288, 4096
    W = O.gaussian_bf16((N, K), 0.02, 7).to(dev)
    for M in (1, 3, 4, 9):                        # 9 rows: the layer falls back to the two launches
        gu = (torch.randn((M, 2 * K), generator=torch.Generator().manual_seed(M)) * 2).to(torch.bfloat16).to(dev)
        act = ops.bi_silu_mul(gu)
        want = matmul_tp_persistent(act, W.t())
        for tp in (1, 2, 4, 8):
            layer = SimulatedTPRowLinear(W, tp)
            assert torch.equal(layer.forward_gated(gu), want), (M, tp)
            assert torch.equal(layer(act), want), (M, tp)
    # shapes the one-launch kernel declines: too many rows; so many activations that forming them in every work-group
    # costs more than a launch of its own (4 rows of 12288); more strips than CUs
    s = torch.cuda.current_stream().cuda_stream
    gu = torch.zeros((5, 2 * K), dtype=torch.bfloat16, device=dev)
    C = torch.empty((5, N), dtype=torch.bfloat16, device=dev)
    L = _lib.lib()
    for rows in (5, 4):
        assert L.tbik_gemm_silu_mul_bf16(gu.data_ptr(), gu.data_ptr() + 2 * K, 2 * K, W.data_ptr(), 1, K, C.data_ptr(), N, rows, N, K,
                                         256, None, s) == _lib.TBIK_ERR_UNSUPPORTED
    Wwide = torch.zeros((8192, 4096), dtype=torch.bfloat16, device=dev)
    Cw = torch.empty((1, 8192), dtype=torch.bfloat16, device=dev)
    assert L.tbik_gemm_silu_mul_bf16(gu.data_ptr(), gu.data_ptr() + 4096, 2 * K, Wwide.data_ptr(), 1, 4096, Cw.data_ptr(), 8192, 1,
                                     8192, 4096, 256, None, s) == _lib.TBIK_ERR_UNSUPPORTED
    W2 = O.gaussian_bf16((5120, 3200), 0.02, 8).to(dev)
    gu2 = (torch.randn((2, 6400), generator=torch.Generator().manual_seed(1))).to(torch.bfloat16).to(dev)
    got = ops.gemm_tree_silu_mul(gu2[:, :3200], gu2[:, 3200:], W2.t(), None, 128)
    assert torch.equal(got, matmul_tp_persistent(ops.bi_silu_mul(gu2), W2.t(), leaf_k=128))


SMALL = DecoderConfig(vocab_size=3000, hidden_size=1024, num_layers=2, num_q_heads=16, num_kv_heads=4, head_dim=128,
                      intermediate_size=4096)


def test_decoder_with_and_without_fused_producers_gives_the_same_bits(dev):
    g = torch.Generator().manual_seed(3)
    prompts = [torch.randint(0, SMALL.vocab_size, (n,), generator=g).tolist() for n in (37, 5, 64, 21, 33, 16, 50, 48)]
    for tp in (1, 2, 8):
        fused = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev, fused_producers=True)
        plain = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev, fused_producers=False)
        for batch in (1, 3, 4, 8):
            print("case decoder fused producers tp", tp, "batch", batch, flush=True)
            a_ids, a_log = fused.generate(prompts[:batch], 6, return_logits=True)
            b_ids, b_log = plain.generate(prompts[:batch], 6, return_logits=True)
            assert torch.equal(a_ids, b_ids) and torch.equal(a_log, b_log), (tp, batch)
        del fused, plain
