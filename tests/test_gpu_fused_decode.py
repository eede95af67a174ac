"""One-launch compositions for decode-sized batches against the two-launch forms they stand for (bit for bit) and
against the CPU oracle: RMSNorm inside the batch-invariant mm (`bi_rmsnorm_gemm_bf16`), SiLU * up inside the tree
matmul of down_proj (`tbik_gemm_silu_mul_bf16`), the add-RMSNorm behind a row-split layer inside the launch that combines
the layer's K shards (`tbik_gemm_rmsnorm_bf16`, `tbik_tree_combine_rmsnorm_bf16`), SiLU * up inside the merged gate/up projection
(`bi_gemm_silu_mul_bf16`)."""
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


@pytest.mark.parametrize("M,K,N,leaf", [(1, 12288, 4096, 256), (2, 8192, 4096, 256), (2, 1536, 4096, 256), (2, 6144, 4096, 256),
                                        (1, 4096, 4096, 256), (2, 3072, 2048, 128), (4, 4096, 4096, 256), (4, 3072, 4096, 256)])
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
    # costs more than a launch of its own (from two rows of 12288 on); more strips than CUs
    s = torch.cuda.current_stream().cuda_stream
    gu = torch.zeros((5, 2 * K), dtype=torch.bfloat16, device=dev)
    C = torch.empty((5, N), dtype=torch.bfloat16, device=dev)
    L = _lib.lib()
    for rows in (5, 4, 2):
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
        plain = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev, fused_producers=False, fused_consumers=False)
        for batch in (1, 3, 4, 8):
            print("case decoder fused producers tp", tp, "batch", batch, flush=True)
            a_ids, a_log = fused.generate(prompts[:batch], 6, return_logits=True)
            b_ids, b_log = plain.generate(prompts[:batch], 6, return_logits=True)
            assert torch.equal(a_ids, b_ids) and torch.equal(a_log, b_log), (tp, batch)
        del fused, plain


def _raw_gemm_rmsnorm(A, W, leaf, bias, res, w, eps, rout, out):
    L = _lib.lib()
    M, K = A.shape
    N = W.shape[0]
    ws_bytes = L.tbik_gemm_workspace_bytes(M, N, K, leaf)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=A.device)
    p = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    return L.tbik_gemm_rmsnorm_bf16(A.data_ptr(), A.stride(0), W.data_ptr(), 1, W.stride(0), M, N, K, leaf, p(bias), p(res),
                                    0 if res is None else res.stride(0), p(w), eps, p(rout), 0 if rout is None else rout.stride(0),
                                    out.data_ptr(), out.stride(0), ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)


@pytest.mark.parametrize("M,K,N,leaf", [(5, 4096, 4096, 256), (32, 12288, 4096, 256), (128, 4096, 4096, 256), (77, 12288, 4096, 256),
                                        (64, 8192, 5120, 256), (16, 6400, 5120, 128), (200, 4096, 1024, 256), (24, 4096, 8192, 256)])
def test_add_rmsnorm_inside_the_shard_combine_of_the_tree_matmul_equals_the_two_calls(dev, M, K, N, leaf):
    A = O.gaussian_bf16((M, K), 1.0, 40 + M).to(dev)
    W = O.gaussian_bf16((N, K), 0.02, 41).to(dev)
    res = O.gaussian_bf16((M, N), 1.0, 42 + M).to(dev)
    w = (1.0 + 0.1 * torch.randn(N, generator=torch.Generator().manual_seed(5))).to(torch.bfloat16).to(dev)
    bias = O.gaussian_bf16((N,), 0.5, 43).to(dev)
    print("case tree matmul + add-rmsnorm", M, K, N, leaf, flush=True)
    plan = (torch.zeros(5, dtype=torch.int32)).numpy()
    import ctypes
    assert _lib.lib().tbik_gemm_plan_info(M, N, K, leaf, 0, 0, plan.ctypes.data_as(ctypes.POINTER(ctypes.c_int))) == 0
    assert plan[0] in (1, 3) and plan[1] > 1, plan          # a shape whose matmul ends in one shard combine
    y = matmul_tp_persistent(A, W.t(), leaf_k=leaf)
    for b in (None, bias):
        yb = y if b is None else ops.gemm_tree(A, W.t(), b, leaf)
        for r in (None, res):
            for nw in (w, None):
                want, want_res = bio.rms_norm(yb, nw, 1e-6, residual=r) if r is not None else (bio.rms_norm(yb, nw, 1e-6), None)
                out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
                rout = None if r is None else torch.empty_like(out)
                assert _raw_gemm_rmsnorm(A, W, leaf, b, r, nw, 1e-6, rout, out) == _lib.TBIK_OK
                assert torch.equal(out, want), (b is None, r is None, nw is None)
                assert r is None or torch.equal(rout, want_res)
                got, got_res = ops.gemm_tree_add_rmsnorm(A, W.t(), b, leaf, r, nw, 1e-6)
                assert torch.equal(got, want) and (r is None or torch.equal(got_res, want_res))
    # the new residual may be written over the old one
    r2 = res.clone()
    out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    assert _raw_gemm_rmsnorm(A, W, leaf, None, r2, w, 1e-6, r2, out) == _lib.TBIK_OK
    want, want_res = bio.rms_norm(y, w, 1e-6, residual=res)
    assert torch.equal(out, want) and torch.equal(r2, want_res)
    # and the whole against the oracle's norm of the oracle-checked product (rounding points as documented: within 2 ulp)
    ref, ref_res = O.rmsnorm(y.cpu(), w.cpu(), 1e-6, residual=res.cpu())
    assert torch.equal(r2.cpu(), ref_res) and O.bf16_ulp_distance(out.cpu(), ref).max() <= 2


def test_add_rmsnorm_behind_the_tree_matmul_falls_back_where_there_is_no_shard_combine(dev):
    W = O.gaussian_bf16((4096, 4096), 0.02, 50).to(dev)
    w = torch.ones(4096, dtype=torch.bfloat16, device=dev)
    for M in (1, 4, 4096):                 # the one-launch few-rows kernel; a grid that needs no K split
        A = O.gaussian_bf16((M, 4096), 1.0, 51).to(dev)
        res = O.gaussian_bf16((M, 4096), 1.0, 52).to(dev)
        out = torch.empty((M, 4096), dtype=torch.bfloat16, device=dev)
        rout = torch.empty_like(out)
        rc = _raw_gemm_rmsnorm(A, W, 256, None, res, w, 1e-6, rout, out)
        want, want_res = bio.rms_norm(matmul_tp_persistent(A, W.t()), w, 1e-6, residual=res)
        if rc != _lib.TBIK_OK:
            assert rc == _lib.TBIK_ERR_UNSUPPORTED, (M, rc)
        else:
            assert torch.equal(out, want) and torch.equal(rout, want_res), M
        got, got_res = ops.gemm_tree_add_rmsnorm(A, W.t(), None, 256, res, w, 1e-6)
        assert torch.equal(got, want) and torch.equal(got_res, want_res), M
    assert _raw_gemm_rmsnorm(O.gaussian_bf16((1, 4096), 1.0, 53).to(dev), W, 256, None, None, w, 1e-6, None,
                             torch.empty((1, 4096), dtype=torch.bfloat16, device=dev)) == _lib.TBIK_ERR_UNSUPPORTED


@pytest.mark.parametrize("rows,hidden,nparts", [(1, 4096, 2), (33, 4096, 8), (7, 1024, 4), (5, 8192, 2), (130, 1000, 4), (3, 5120, 32)])
def test_add_rmsnorm_inside_the_shard_combine_equals_the_separate_calls(dev, rows, hidden, nparts):
    parts = [O.gaussian_bf16((rows, hidden), 1.0, 60 + i).to(dev) for i in range(nparts)]
    res = O.gaussian_bf16((rows, hidden), 1.0, 59).to(dev)
    w = (1.0 + 0.1 * torch.randn(hidden, generator=torch.Generator().manual_seed(6))).to(torch.bfloat16).to(dev)
    bias = O.gaussian_bf16((hidden,), 0.5, 58).to(dev)
    print("case shard combine + add-rmsnorm", rows, hidden, nparts, flush=True)
    y = ops.tree_combine(parts)
    assert torch.equal(y.cpu(), O.tree_combine([p.cpu() for p in parts]))
    for b in (None, bias):
        yb = y if b is None else y + b
        for r in (None, res):
            want, want_res = bio.rms_norm(yb, w, 1e-6, residual=r) if r is not None else (bio.rms_norm(yb, w, 1e-6), None)
            got, got_res = ops.tree_combine_add_rmsnorm(parts, b, r, w, 1e-6)
            assert torch.equal(got, want), (b is None, r is None)
            assert r is None or torch.equal(got_res, want_res)
    # what the one-launch kernel does not take goes through the separate calls (fp16 partials here)
    half = [O.gaussian_bf16((2, 512), 1.0, 70 + i).to(torch.float16).to(dev) for i in range(2)]
    g, _ = ops.tree_combine_add_rmsnorm(half, None, None, None, 1e-6)
    assert torch.equal(g, bio.rms_norm(ops.tree_combine(half), None, 1e-6))


def test_decoder_with_and_without_fused_consumers_gives_the_same_bits(dev):
    g = torch.Generator().manual_seed(4)
    prompts = [torch.randint(0, SMALL.vocab_size, (n,), generator=g).tolist() for n in (37, 5, 64, 21, 33, 16, 50, 48, 9, 12)]
    for tp in (1, 2, 4):
        fused = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev, fused_consumers=True)
        plain = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev, fused_consumers=False)
        for batch in (1, 5, 10):
            print("case decoder fused consumers tp", tp, "batch", batch, flush=True)
            a_ids, a_log = fused.generate(prompts[:batch], 6, return_logits=True)
            b_ids, b_log = plain.generate(prompts[:batch], 6, return_logits=True)
            assert torch.equal(a_ids, b_ids) and torch.equal(a_log, b_log), (tp, batch)
        del fused, plain


@pytest.mark.parametrize("M,K,inter", [(5, 4096, 12288), (16, 4096, 12288), (17, 4096, 12288), (32, 4096, 12288), (33, 4096, 12288),
                                       (64, 4096, 12288), (40, 1024, 4096), (9, 5120, 3200), (48, 2048, 2064), (12, 8192, 1024)])
def test_silu_mul_inside_the_merged_projection_equals_the_two_calls(dev, M, K, inter):
    x = O.gaussian_bf16((M, K), 1.0, 80 + M).to(dev)
    W = O.gaussian_bf16((2 * inter, K), 0.03, 81).to(dev)
    print("case mm + silu_mul", M, K, inter, flush=True)
    want = ops.bi_silu_mul(bio.matmul_persistent(x, W.t()))
    out = torch.empty((M, inter), dtype=torch.bfloat16, device=dev)
    s = torch.cuda.current_stream().cuda_stream
    L = _lib.lib()
    # the raw entry point takes the shape (so the wrapper below did not fall back to the two calls)
    assert L.bi_gemm_silu_mul_bf16(x.data_ptr(), K, W.data_ptr(), K, out.data_ptr(), inter, M, inter, K, s) == _lib.TBIK_OK
    assert torch.equal(out, want)
    assert torch.equal(ops.gemm_silu_mul(x, W), want)
    # activations and output as views with a row stride of their own
    xp = torch.zeros((M, K + 64), dtype=torch.bfloat16, device=dev)
    xp[:, :K] = x
    op = torch.zeros((M, inter + 8), dtype=torch.bfloat16, device=dev)
    assert L.bi_gemm_silu_mul_bf16(xp.data_ptr(), K + 64, W.data_ptr(), K, op.data_ptr(), inter + 8, M, inter, K, s) == _lib.TBIK_OK
    assert torch.equal(op[:, :inter], want) and (op[:, inter:] == 0).all()
    # every row alone gives the row of the batch (batch invariance of the fused form; a single row takes the two calls)
    assert torch.equal(ops.gemm_silu_mul(x[M - 1:], W)[0], want[M - 1])
    # and the oracle's activation of the kernel's own product (the product itself is oracle-checked elsewhere)
    assert O.bf16_ulp_distance(out.cpu(), O.silu_mul(bio.matmul_persistent(x, W.t()).cpu())).max() <= 1


def test_silu_mul_inside_the_merged_projection_declines_other_row_counts(dev):
    W = O.gaussian_bf16((2 * 4096, 1024), 0.03, 82).to(dev)
    s = torch.cuda.current_stream().cuda_stream
    for M, inter in ((4, 4096), (1, 4096), (65, 4096), (300, 4096), (20, 4088)):     # few rows, many rows, a ragged strip
        x = O.gaussian_bf16((M, 1024), 1.0, 83).to(dev)
        out = torch.empty((M, inter), dtype=torch.bfloat16, device=dev)
        assert _lib.lib().bi_gemm_silu_mul_bf16(x.data_ptr(), 1024, W.data_ptr(), 1024, out.data_ptr(), inter, M, inter, 1024, s) \
            == _lib.TBIK_ERR_UNSUPPORTED, (M, inter)
        if inter == 4096:
            assert torch.equal(ops.gemm_silu_mul(x, W), ops.bi_silu_mul(bio.matmul_persistent(x, W.t())))


def test_decoder_at_forty_sequences_with_and_without_fused_consumers_gives_the_same_bits(dev):
    """40 rows per decode step: the add-RMSNorm inside the shard combines and SiLU * up inside the merged projection."""
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, SMALL.vocab_size, (int(n),), generator=g).tolist() for n in torch.randint(3, 20, (40,), generator=g)]
    fused = Qwen3Decoder(SMALL, tp_size=1, seed=0, device=dev, fused_consumers=True)
    plain = Qwen3Decoder(SMALL, tp_size=1, seed=0, device=dev, fused_consumers=False, fused_attention_step=False)
    a_ids, a_log = fused.generate(prompts, 5, return_logits=True)
    b_ids, b_log = plain.generate(prompts, 5, return_logits=True)
    assert torch.equal(a_ids, b_ids) and torch.equal(a_log, b_log)
