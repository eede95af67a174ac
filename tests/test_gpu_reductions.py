"""GPU parity and batch invariance of RMSNorm, log_softmax / softmax, mean and the single-accumulator mm."""
import math

import pytest
import torch

from oracle import tbik_oracle as O
from llm_reproducibility_amd.bio import batch_invariant_ops as bio

pytestmark = pytest.mark.gpu
ROWS = (1, 7, 256, 4096)


def test_rmsnorm_parity_and_batch_invariance(dev):
    x = O.gaussian_bf16((4096, 4096), 1.0, 0)
    w = (1.0 + 0.1 * torch.randn(4096, generator=torch.Generator().manual_seed(1))).to(torch.bfloat16)
    xd, wd = x.to(dev), w.to(dev)
    full = bio.rms_norm(xd, wd, 1e-6)
    want = O.rmsnorm(x[:300], w, 1e-6)
    # stated tolerance: within 1 bf16 ulp of the oracle OR within 2^-8 of the output scale.  The kernel's fp32 sum of
    # squares runs in another order than the CPU's, so the normalised value may land on the other side of a rounding
    # boundary (1 ulp); the bf16 multiply by the weight can carry that step into the binade below, where the same
    # absolute step counts as 2 ulp -- never more, and only on a small fraction of the elements.
    assert not O.outside_tolerance(full[:300], want).any()
    ulp = O.bf16_ulp_distance(full[:300].cpu(), want)
    assert ulp.max() <= 2 and (ulp > 0).float().mean() < 0.02 and (ulp > 1).float().mean() < 1e-3, \
        (ulp.max(), (ulp > 0).float().mean(), (ulp > 1).float().mean())
    for r in ROWS:
        assert torch.equal(bio.rms_norm(xd[:r], wd, 1e-6), full[:r]), r
    assert torch.equal(bio.rms_norm(xd[1234:1235], wd, 1e-6), full[1234:1235])
    # exact case: +-1 row with unit weight
    s = torch.ones((3, 4096), dtype=torch.bfloat16)
    s[:, ::2] = -1
    assert torch.equal(bio.rms_norm(s.to(dev), torch.ones(4096, dtype=torch.bfloat16, device=dev), 1e-6).cpu(), s)


def test_rmsnorm_rounding_points_on_an_exact_case(dev):
    """The case of tests/test_oracle_reductions.py whose normalisation factor is exactly 1/3 (integer squares: the
    sum is exact in any order), so the kernel has to give the bits of exact rational arithmetic with the documented
    rounding points -- the normalised value rounded to bf16 BEFORE the bf16 multiply by the weight -- and not those of a
    single rounding after an fp32 multiply."""
    from test_oracle_reductions import rounding_point_case
    x, w, two_roundings, one_rounding = rounding_point_case()
    got = bio.rms_norm(x.to(dev), w.to(dev), 0.0).cpu()
    assert torch.equal(got, two_roundings)
    assert (got != one_rounding).sum() > 100
    half = (x.float() / 2).to(torch.bfloat16)
    y, new_res = bio.rms_norm(half.to(dev), w.to(dev), 0.0, residual=half.to(dev))
    assert torch.equal(new_res.cpu(), x) and torch.equal(y.cpu(), two_roundings)
    rows = x.repeat(300, 1)
    assert torch.equal(bio.rms_norm(rows.to(dev), w.to(dev), 0.0).cpu(), two_roundings.repeat(300, 1))


def test_fp16_rmsnorm_and_silu_mul(dev):
    from llm_reproducibility_amd import ops
    x = O.gaussian_bf16((300, 4096), 1.0, 0).to(torch.float16)
    r = O.gaussian_bf16((300, 4096), 1.0, 3).to(torch.float16)
    w = (1.0 + 0.1 * torch.randn(4096, generator=torch.Generator().manual_seed(1))).to(torch.float16)
    got = bio.rms_norm(x.to(dev), w.to(dev), 1e-6)
    want = O.rmsnorm(x, w, 1e-6)
    assert got.dtype == torch.float16
    assert ((got.cpu().float() - want.float()).abs() <= 2.0 ** -9 * want.float().abs().clamp_min(2.0 ** -4)).all()
    g2, res2 = bio.rms_norm(x.to(dev), w.to(dev), 1e-6, residual=r.to(dev))
    w2, wres = O.rmsnorm(x, w, 1e-6, residual=r)
    assert torch.equal(res2.cpu(), wres)
    assert ((g2.cpu().float() - w2.float()).abs() <= 2.0 ** -9 * w2.float().abs().clamp_min(2.0 ** -4)).all()
    for rows in (1, 7, 64):
        assert torch.equal(bio.rms_norm(x[:rows].to(dev), w.to(dev), 1e-6), got[:rows])
    gu = (torch.randn((65, 2 * 1024), generator=torch.Generator().manual_seed(2)) * 2).to(torch.float16)
    act = ops.bi_silu_mul(gu.to(dev))
    wa = O.silu_mul(gu)
    assert act.dtype == torch.float16
    assert ((act.cpu().float() - wa.float()).abs() <= 2.0 ** -9 * wa.float().abs().clamp_min(2.0 ** -6)).all()
    assert torch.equal(ops.bi_silu_mul(gu[:3].to(dev)), act[:3])


def test_add_rmsnorm_parity(dev):
    x = O.gaussian_bf16((64, 4096), 1.0, 2)
    res = O.gaussian_bf16((64, 4096), 1.0, 3)
    w = O.gaussian_bf16((4096,), 1.0, 4)
    out, new_res = bio.rms_norm(x.to(dev), w.to(dev), 1e-6, residual=res.to(dev))
    want, want_res = O.rmsnorm(x, w, 1e-6, residual=res)
    assert torch.equal(new_res.cpu(), want_res)
    assert not O.outside_tolerance(out, want).any() and O.bf16_ulp_distance(out.cpu(), want).max() <= 2
    for hidden in (8, 64, 520, 1024, 5120, 8192):
        xs = O.gaussian_bf16((5, hidden), 2.0, hidden)
        ws = O.gaussian_bf16((hidden,), 1.0, hidden + 1)
        got = bio.rms_norm(xs.to(dev), ws.to(dev), 1e-5)
        ws_want = O.rmsnorm(xs, ws, 1e-5)
        assert not O.outside_tolerance(got, ws_want).any() and O.bf16_ulp_distance(got.cpu(), ws_want).max() <= 2, hidden


def test_log_softmax_parity_and_batch_invariance(dev):
    V = 151936
    g = torch.Generator().manual_seed(0)
    x = torch.randn((256, V), generator=g) * 3.0
    xd = x.to(dev)
    full = bio.log_softmax(xd)
    want = torch.log_softmax(x[:16].double(), dim=-1)
    assert (full[:16].cpu().double() - want).abs().max() < 2e-5
    for r in (1, 7, 256):
        assert torch.equal(bio.log_softmax(xd[:r]), full[:r]), r
    assert torch.equal(bio.log_softmax(xd[100:101]), full[100:101])
    big = xd.repeat(16, 1)                                   # 4096 rows
    out_big = bio.log_softmax(big)
    assert torch.equal(out_big[:256], full) and torch.equal(out_big[-256:], full)
    # softmax = exp(log_softmax), sums to 1
    sm = bio.softmax(xd[:7])
    assert (sm.sum(-1) - 1).abs().max() < 1e-4
    assert (sm.cpu().double() - torch.softmax(x[:7].double(), -1)).abs().max() < 1e-6
    # closed forms: constant row -> -log V; ragged widths incl. not a multiple of 4
    c = torch.full((2, 1000), 4.25, device=dev)
    assert torch.allclose(bio.log_softmax(c), torch.full_like(c, -math.log(1000.0)), atol=2e-6)
    for cols in (1, 3, 5, 4095, 4096, 4097, 8191, 12289):
        y = torch.randn((3, cols), generator=g)
        got = bio.log_softmax(y.to(dev)).cpu()
        assert (got.double() - torch.log_softmax(y.double(), -1)).abs().max() < 1e-5, cols
    # bf16 input keeps its dtype
    yb = torch.randn((4, 512), generator=g).to(torch.bfloat16)
    assert bio.log_softmax(yb.to(dev)).dtype == torch.bfloat16


def test_log_softmax_4096_distinct_rows_against_fp64(dev):
    """The largest reduction of the benchmark configuration with every row different: 4096 x 151936 fp32 logits
    drawn on the GPU (2.5 GB), float64 parity on 64 rows spread over the whole batch (first, last, and a stride that
    is odd so that every XCD's share of the rows is sampled), and those rows alone / in small batches bit for bit."""
    V, R = 151936, 4096
    g = torch.Generator(device=dev).manual_seed(11)
    x = torch.randn((R, V), generator=g, device=dev) * 3.0
    out = bio.log_softmax(x)
    pick = sorted(set([0, 1, R - 2, R - 1] + [(61 * i + 17) % R for i in range(60)]))
    idx = torch.tensor(pick, device=dev)
    want = torch.log_softmax(x[idx].cpu().double(), dim=-1)
    got = out[idx].cpu().double()
    assert (got - want).abs().max() < 2e-5, (got - want).abs().max()
    assert not torch.equal(out[0], out[1])
    for r in (0, 777, R - 1):                                        # a row alone (two-launch schedule)
        assert torch.equal(bio.log_softmax(x[r:r + 1]), out[r:r + 1]), r
    assert torch.equal(bio.log_softmax(x[2000:2007]), out[2000:2007])
    assert torch.equal(bio.log_softmax(x[1024:1280]), out[1024:1280])   # 256 rows: the resident schedule again
    del x, out
    torch.cuda.empty_cache()


def test_log_softmax_of_offset_logits(dev):
    """log_softmax(x + c) = log_softmax(x): with the difference to the maximum formed before the scaling by log2(e) a
    common offset costs only the rounding of x + c itself.  Logits around +1000 and -1e4 against float64 of the same
    fp32 values; the tolerance is that of the unshifted test (2e-5) -- a kernel that folds max * log2(e) into a fused
    multiply-add is off by 3e-4 at |max| = 1e4."""
    g = torch.Generator().manual_seed(12)
    base = torch.randn((200, 151936), generator=g) * 3.0
    for shift in (1000.0, -1.0e4):
        x = base + shift                                             # rounded to fp32 here, on both sides alike
        got = bio.log_softmax(x.to(dev))
        want = torch.log_softmax(x[:8].double(), dim=-1)
        assert (got[:8].cpu().double() - want).abs().max() < 2e-5, (shift, (got[:8].cpu().double() - want).abs().max())
        assert torch.equal(bio.log_softmax(x[:3].to(dev)), got[:3]), shift      # both schedules


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_log_softmax_reads_16_bit_logits_in_the_kernel(dev, dtype):
    """bf16 / fp16 logits go to the kernel as they are (no fp32 copy in front): result = the fp64 log_softmax of the
    16-bit values rounded once to the output type; half_to_float gives the fp32 result of the same arithmetic; rows
    alone, in a small batch (two launches) and in a large one (row resident on chip) agree bit for bit."""
    from llm_reproducibility_amd import ops
    V = 151936
    g = torch.Generator().manual_seed(3)
    x = (torch.randn((200, V), generator=g) * 3.0).to(dtype)
    xd = x.to(dev)
    full = bio.log_softmax(xd)                       # 200 rows: resident schedule
    assert full.dtype == dtype
    want = torch.log_softmax(x[:8].double(), dim=-1)
    f32 = ops.bi_log_softmax(xd, False, True)
    assert f32.dtype == torch.float32 and (f32[:8].cpu().double() - want).abs().max() < 2e-5
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11       # one unit in the last place, relative
    assert ((full[:8].cpu().double() - want).abs() <= eps * want.abs() + 1e-6).all()
    assert torch.equal(full, f32.to(dtype))          # the 16-bit output is the fp32 result rounded once
    for r in (1, 7, 191, 192):
        assert torch.equal(bio.log_softmax(xd[:r]), full[:r]), r
    assert torch.equal(bio.log_softmax(xd[100:101]), full[100:101])
    sm = ops.bi_log_softmax(xd[:5], True, True)
    assert (sm.cpu().double() - torch.softmax(x[:5].double(), -1)).abs().max() < 1e-6
    # strided rows (a column block of a wider tensor), misaligned start, ragged width
    wide = (torch.randn((260, 5003), generator=g)).to(dtype).to(dev)
    view = wide[:, 3:5000]
    got = bio.log_softmax(view)
    assert ((got.cpu().double() - torch.log_softmax(view.cpu().double(), -1)).abs() <= eps * 12 + 1e-6).all()
    assert torch.equal(got[:3], bio.log_softmax(view[:3]))


def test_log_softmax_schedules_agree_on_widths_around_the_resident_limit(dev):
    """fp32, 200 rows (one launch, row on chip) against the same rows in batches of 3 (two launches): same bits for
    widths that end inside the register part, inside the LDS part, on the limit, and beyond it (two launches again)."""
    g = torch.Generator().manual_seed(5)
    for cols in (4096, 114688, 114689, 130001, 154624, 154625):
        x = (torch.randn((200, cols), generator=g) * 2.0).to(dev)
        big = bio.log_softmax(x)
        for r0 in (0, 77, 197):
            assert torch.equal(bio.log_softmax(x[r0:r0 + 3]), big[r0:r0 + 3]), (cols, r0)
        want = torch.log_softmax(x[:2].cpu().double(), -1)
        assert (big[:2].cpu().double() - want).abs().max() < 2e-5, cols
        del x, big


def test_mean_parity_and_batch_invariance(dev):
    g = torch.Generator().manual_seed(0)
    x = torch.randn((4096, 4096), generator=g)
    xd = x.to(dev)
    full = bio.mean_dim(xd, -1)
    assert (full.cpu().double() - x.double().mean(-1)).abs().max() < 1e-6
    for r in ROWS:
        assert torch.equal(bio.mean_dim(xd[:r], -1), full[:r]), r
    ints = torch.arange(0, 4096, dtype=torch.float32, device=dev).repeat(3, 1)
    assert torch.equal(bio.mean_dim(ints, 1, keepdim=True), torch.full((3, 1), 2047.5, device=dev))
    # long rows (block-per-row), a middle dimension, bf16
    y = torch.randn((5, 20000), generator=g)
    assert (bio.mean_dim(y.to(dev), 1).cpu().double() - y.double().mean(1)).abs().max() < 1e-6
    z = torch.randn((6, 37, 10), generator=g)
    assert (bio.mean_dim(z.to(dev), 1).cpu().double() - z.double().mean(1)).abs().max() < 1e-6
    zb = z.to(torch.bfloat16)
    got = bio.mean_dim(zb.to(dev), 2)
    assert got.dtype == torch.bfloat16 and (got.cpu().float() - zb.float().mean(2)).abs().max() < 1e-2


def test_single_accumulator_mm_parity_and_batch_invariance(dev):
    a = O.gaussian_bf16((300, 4096), 1.0, 0)
    w = O.gaussian_bf16((1000, 4096), 0.02, 1)                # [N,K] as nn.Linear stores it
    bias = O.gaussian_bf16((1000,), 1.0, 2)
    ad, wd, bd = a.to(dev), w.to(dev), bias.to(dev)
    full = bio.matmul_persistent(ad, wd.t(), bd)
    want = O.matmul_single_acc(a, w.t(), bias)
    assert not O.outside_tolerance(full, want).any()
    assert (O.bf16_ulp_distance(full.cpu(), want) > 0).float().mean() < 0.02
    for m in (1, 7, 64, 129):
        assert torch.equal(bio.matmul_persistent(ad[:m], wd.t(), bd), full[:m]), m
    # exact on integers, K not a multiple of 64 nor of 8, row-major b
    ai = O.integer_bf16((33, 1003), -9, 9, 3)
    bi = O.integer_bf16((1003, 40), -7, 7, 4)
    got = bio.matmul_persistent(ai.to(dev), bi.to(dev))
    assert torch.equal(got.cpu(), O.matmul_single_acc(ai, bi))


def test_single_accumulator_mm_large_and_small_kernels_agree_bitwise(dev):
    # M=2048 takes the wide pipeline, M<=64 the streaming kernels, M=300 the tiled one: same MFMA chain per element, same bits
    a = O.gaussian_bf16((2048, 1024), 1.0, 5)
    w = O.gaussian_bf16((4096, 1024), 0.05, 6)
    bias = O.gaussian_bf16((4096,), 1.0, 7)
    ad, wd, bd = a.to(dev), w.to(dev), bias.to(dev)
    full = bio.matmul_persistent(ad, wd.t(), bd)
    for m in (1, 3, 16, 17, 32, 33, 48, 64, 128, 300):  # streaming kernels, the one-round 128-row tiles (33..128), the tiled one
        assert torch.equal(bio.matmul_persistent(ad[:m], wd.t(), bd), full[:m]), m
    want = O.matmul_single_acc(a[:256], w.t(), bias)
    assert not O.outside_tolerance(full[:256], want).any()
    ai = O.integer_bf16((2048, 512), -9, 9, 8)
    wi = O.integer_bf16((4096, 512), -7, 7, 9)
    assert torch.equal(bio.matmul_persistent(ai.to(dev), wi.to(dev).t()).cpu(), O.matmul_single_acc(ai, wi.t()))


def test_single_accumulator_mm_on_narrow_weight_matrices_equals_its_small_pieces(dev):
    """Fewer than 4096 weight rows (a TP shard of a column-split layer) at 33 .. 128 activation rows take the 128-row tiles
    at the width a cost model picks, and from 64 rows on a grid of at most 128 such tiles (4096 weight rows included) is
    cut into tiles that own 64 or 32 of their rows: same bits as 16 rows at a time through the streaming kernels, ragged
    widths and a bias included, and within the tolerance of the CPU oracle."""
    for N, K in ((512, 4096), (768, 1024), (1000, 2048), (2048, 6144), (3072, 1024), (3584, 512), (4096, 1024)):
        w = O.gaussian_bf16((N, K), 0.05, N + K).to(dev)
        bias = O.gaussian_bf16((N,), 1.0, N).to(dev)
        a = O.gaussian_bf16((128, K), 1.0, K).to(dev)
        pieces = torch.cat([bio.matmul_persistent(a[r:r + 16], w.t(), bias) for r in range(0, 128, 16)])
        for m in (33, 48, 64, 65, 100, 128):
            print("case narrow mm", m, N, K, flush=True)
            assert torch.equal(bio.matmul_persistent(a[:m], w.t(), bias), pieces[:m]), (m, N, K)
        assert torch.equal(bio.matmul_persistent(a[:100], w.t()), torch.cat([bio.matmul_persistent(a[r:r + 4], w.t()) for r in range(0, 100, 4)]))
    a = O.gaussian_bf16((100, 1024), 1.0, 3)
    w = O.gaussian_bf16((768, 1024), 0.05, 4)
    assert not O.outside_tolerance(bio.matmul_persistent(a.to(dev), w.to(dev).t()), O.matmul_single_acc(a, w.t())).any()


def test_single_accumulator_mm_every_shape_of_a_sweep_equals_its_small_pieces(dev):
    """The mm picks among six kernel families and a dozen tile widths from measured cost models; none of it may change a
    bit.  Over a seeded sweep of shapes (rows 1 .. 4096, the projection widths of the 8B and 32B configurations and ragged
    ones, K a multiple of 64, of 32 and of 8 only) the product equals the same product computed in pieces of 16 rows by
    128 columns, which the streaming kernels serve."""
    g = torch.Generator().manual_seed(11)
    Ms = (1, 5, 16, 31, 33, 64, 65, 100, 128, 129, 200, 256, 300, 512, 777, 1024, 1536, 2048, 4096)
    Ns = (128, 1000, 1024, 3072, 4096, 5120, 6144, 8192, 10240, 24576)
    Ks = (256, 320, 520, 1024, 2048, 4096, 5120)
    picks = set()
    while len(picks) < 48:
        picks.add((Ms[int(torch.randint(len(Ms), (1,), generator=g))], Ns[int(torch.randint(len(Ns), (1,), generator=g))],
                   Ks[int(torch.randint(len(Ks), (1,), generator=g))]))
    for M, N, K in sorted(picks):
        if M * N * K > 6e10:
            continue
        print("case mm sweep", M, N, K, flush=True)
        A = O.gaussian_bf16((M, K), 1.0, M + N).to(dev)
        Wt = O.gaussian_bf16((N, K), 0.02, K).to(dev).t()
        got = bio.matmul_persistent(A, Wt)
        # pieces: 16 rows (all rows of a small batch at once) by 128 columns
        rows = range(0, M, 16) if M <= 64 else [int(r) for r in torch.randint(0, M - 15, (4,), generator=g)]
        for m0 in rows:
            m1 = min(M, m0 + 16)
            for n0 in range(0, N, 1024 if N > 2048 else 128):
                piece = bio.matmul_persistent(A[m0:m1], Wt[:, n0:n0 + 128])
                assert torch.equal(piece, got[m0:m1, n0:n0 + 128]), (M, N, K, m0, n0)


# (M, N, K) -> tile width the cost model picks: 64 / 96 / 192 / 128 / 256 / 32 columns, ragged edges in M and N
@pytest.mark.parametrize("M,N,K", [(200, 6144, 1024), (500, 6100, 512), (700, 6144, 1024), (384, 8192, 2048), (1100, 8200, 256),
                                   (130, 40, 512), (257, 24576, 320)])
def test_single_accumulator_mm_balanced_tiles_match_oracle_bitwise(dev, M, N, K):
    """More than 128 rows: 128-row tiles whose width is chosen to spread the grid over the chip.  Integer inputs, so the
    oracle's bits are the only right answer; a row alone (streaming kernel) and inside the batch agree bitwise."""
    print("case", M, N, K, flush=True)
    a = O.integer_bf16((M, K), -9, 9, 31)
    w = O.integer_bf16((N, K), -7, 7, 32)
    bias = O.integer_bf16((N,), -5, 5, 33)
    ad, wd, bd = a.to(dev), w.to(dev), bias.to(dev)
    got = bio.matmul_persistent(ad, wd.t(), bd)
    assert torch.equal(got.cpu(), O.matmul_single_acc(a, w.t(), bias))
    assert torch.equal(bio.matmul_persistent(ad[M - 1:M], wd.t(), bd), got[M - 1:M])
    assert torch.equal(bio.matmul_persistent(ad[:129], wd.t(), bd), got[:129])
    g = O.gaussian_bf16((M, K), 1.0, 34)
    gw = O.gaussian_bf16((N, K), 0.05, 35)
    full = bio.matmul_persistent(g.to(dev), gw.to(dev).t())
    assert torch.equal(bio.matmul_persistent(g[:64].to(dev), gw.to(dev).t()), full[:64])
    assert not O.outside_tolerance(full, O.matmul_single_acc(g, gw.t())).any()


# grids of more than one round, where the cost model picks tiles of 256 rows: one round of 256 tiles with ragged edges in
# M and N, an odd number of 64-wide slices, five rounds with a last column of tiles eight columns wide; then 256x192
# tiles (qkv-like: one round of 256 tiles; two rounds; ragged in M and N), 192x192 tiles (gate_up at 384 rows: one round
# of 256 tiles; ragged) and 192x256 tiles (one round of 256 tiles)
@pytest.mark.parametrize("M,N,K", [(2040, 8190, 1024), (4096, 4090, 2112), (8192, 8200, 1024), (2048, 8192, 768),
                                   (2048, 6144, 1024), (4096, 6144, 512), (1990, 6100, 1088),
                                   (384, 24576, 1024), (1530, 6100, 1024), (3072, 4096, 2048)])
def test_single_accumulator_mm_256_tiles_match_oracle_bitwise(dev, M, N, K):
    """256x256 tiles (accumulators pinned by hand in both register files, ten-block LDS ring): integer inputs, so the
    oracle's bits are the only right answer; rows alone (streaming kernel), the first 129 rows (128-row tiles) and the
    whole batch agree bitwise; Gaussian inputs stay inside the tolerance and agree with the 128-row tiles bitwise."""
    print("case", M, N, K, flush=True)
    a = O.integer_bf16((M, K), -9, 9, 41)
    w = O.integer_bf16((N, K), -7, 7, 42)
    bias = O.integer_bf16((N,), -5, 5, 43)
    ad, wd, bd = a.to(dev), w.to(dev), bias.to(dev)
    got = bio.matmul_persistent(ad, wd.t(), bd)
    assert torch.equal(got.cpu(), O.matmul_single_acc(a, w.t(), bias))
    assert torch.equal(bio.matmul_persistent(ad[M - 1:M], wd.t(), bd), got[M - 1:M])
    assert torch.equal(bio.matmul_persistent(ad[:129], wd.t(), bd), got[:129])
    g = O.gaussian_bf16((M, K), 1.0, 44)
    gw = O.gaussian_bf16((N, K), 0.05, 45)
    gd, gwd = g.to(dev), gw.to(dev)
    full = bio.matmul_persistent(gd, gwd.t())
    for lo in range(0, M, 640):  # pieces of at most 640 rows take the 128-row tiles: same MFMA chain, same bits
        assert torch.equal(bio.matmul_persistent(gd[lo:lo + 640], gwd.t()), full[lo:lo + 640]), lo
    assert not O.outside_tolerance(full[:512], O.matmul_single_acc(g[:512], gw.t())).any()
    assert torch.equal(bio.matmul_persistent(gd, gwd.t()), full)  # and the same bits on a second launch


@pytest.mark.parametrize("M,N,K", [(128, 6144, 4096), (65, 8200, 1024), (33, 24576, 512), (100, 16384, 512), (128, 16400, 256), (40, 12296, 1088)])
def test_single_accumulator_mm_one_round_tiles_match_oracle_bitwise(dev, M, N, K):
    """33..128 rows on a grid of 128-row tiles that is resident at once (tile widths 32, 64, 96 and 128, ragged last
    tiles, bias): integer inputs, so the oracle's bits are the only right answer."""
    print("case", M, N, K, flush=True)
    a = O.integer_bf16((M, K), -9, 9, 21)
    w = O.integer_bf16((N, K), -7, 7, 22)
    bias = O.integer_bf16((N,), -5, 5, 23)
    got = bio.matmul_persistent(a.to(dev), w.to(dev).t(), bias.to(dev))
    assert torch.equal(got.cpu(), O.matmul_single_acc(a, w.t(), bias))
    row = bio.matmul_persistent(a[M - 1:M].to(dev), w.to(dev).t(), bias.to(dev))   # the same row through the streaming kernel
    assert torch.equal(row, got[M - 1:M])


def test_single_accumulator_mm_streaming_kernels_on_ragged_shapes(dev):
    # K = 35 steps of 32 (two whole windows and a partial one), N ends inside a 16-wide strip, strided A, bias
    ai = O.integer_bf16((40, 1200), -9, 9, 11)[:, :1120]
    wi = O.integer_bf16((72 + 8, 1120), -7, 7, 12)[:72]
    bi = O.integer_bf16((72,), -5, 5, 13)
    want = O.matmul_single_acc(ai, wi.t(), bi)
    for m in (1, 2, 5, 16, 23, 40):
        got = bio.matmul_persistent(ai[:m].to(dev)[:, :], wi.to(dev).t(), bi.to(dev))
        assert torch.equal(got.cpu(), want[:m]), m
    a_strided = O.integer_bf16((40, 1200), -9, 9, 11).to(dev)[:, :1120]
    assert not a_strided.is_contiguous()
    assert torch.equal(bio.matmul_persistent(a_strided[:5], wi.to(dev).t(), bi.to(dev)).cpu(), want[:5])
    # long K for a single row (the whole-X kernel stages up to 32768 activations)
    a1 = O.integer_bf16((2, 16384), -3, 3, 14)
    w1 = O.integer_bf16((48, 16384), -3, 3, 15)
    assert torch.equal(bio.matmul_persistent(a1.to(dev), w1.to(dev).t()).cpu(), O.matmul_single_acc(a1, w1.t()))


# the windowed streaming kernel forms work-groups of 2, 3, 4, 6 or 8 strips so that every CU gets the same number; with 3
# and 6 the staging loads of a window do not divide among the threads (the last ones repeat the last chunk)
@pytest.mark.parametrize("M,N,K", [(32, 24576, 1024), (20, 12288, 1024), (12, 24576, 4096), (40, 2048, 1024), (17, 18432, 544),
                                   (9, 10240, 4096), (31, 16380, 1056)])
def test_single_accumulator_mm_streaming_kernel_with_balanced_strip_counts(dev, M, N, K):
    print("case", M, N, K, flush=True)
    a = O.integer_bf16((M, K), -9, 9, 300 + M)
    w = O.integer_bf16((N, K), -7, 7, 310 + N % 101)
    bias = O.integer_bf16((N,), -50, 50, 320)
    want = O.matmul_single_acc(a, w.t(), bias)
    got = bio.matmul_persistent(a.to(dev), w.to(dev).t(), bias.to(dev))
    assert torch.equal(got.cpu(), want)
    # a row alone (the whole-X kernel) has the bits it has in the batch
    assert torch.equal(bio.matmul_persistent(a[M - 1:].to(dev), w.to(dev).t(), bias.to(dev)).cpu(), want[M - 1:])


@pytest.mark.parametrize("M,N,K", [(1, 6144, 4096), (5, 1000, 1120), (40, 24576, 512), (64, 1544, 2048), (100, 520, 1024), (300, 4096, 4096)])
def test_single_accumulator_mm_c_abi_strided_and_misaligned_output(dev, M, N, K):
    """bi_gemm_bf16 itself (no wrapper): C is a column block of a wider matrix, then the same block shifted by one
    element (scalar stores): the streaming kernels with 1/3/4/8 strips per work-group, the tiled and the quad kernel."""
    from llm_reproducibility_amd import _lib
    L = _lib.lib()
    print("case", M, N, K, flush=True)
    A = O.integer_bf16((M, K), -9, 9, 3).to(dev)
    W = O.integer_bf16((N, K), -7, 7, 4).to(dev)
    bias = O.integer_bf16((N,), -5, 5, 5).to(dev)
    want = bio.matmul_persistent(A, W.t(), bias)
    assert torch.equal(want[:8].cpu(), O.matmul_single_acc(A[:8].cpu(), W.cpu().t(), bias.cpu()))
    stream = torch.cuda.current_stream().cuda_stream
    for shift in (8, 9):
        wide = torch.full((M, N + 24), 7.0, device=dev, dtype=torch.bfloat16)
        rc = L.bi_gemm_bf16(A.data_ptr(), K, W.data_ptr(), 1, K, wide.data_ptr() + 2 * shift, N + 24, M, N, K, bias.data_ptr(), stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        assert torch.equal(wide[:, shift:shift + N], want), f"shift {shift}"
        assert bool((wide[:, :shift] == 7).all()) and bool((wide[:, shift + N:] == 7).all()), "wrote outside its block"


@pytest.mark.parametrize("M,N,K", [(1, 100, 200), (7, 64, 4096), (33, 1000, 328), (200, 520, 1024)])
def test_single_accumulator_mm_row_major_b_in_place(dev, M, N, K):
    """mm_batch_invariant on a plain row-major [K,N] operand (what `x @ W` hands to the aten override, backward
    matmuls included): no copy of B, integer inputs bit-exact vs the oracle, rows independent of the batch."""
    from llm_reproducibility_amd import _lib
    L = _lib.lib()
    a = O.integer_bf16((M, K), -9, 9, 1)
    bw = O.integer_bf16((K, N + (-N) % 8), -7, 7, 2)
    b = bw[:, :N]
    bias = O.integer_bf16((N,), -300, 300, 3)
    want = O.matmul_single_acc(a, b, bias)
    ad, bd, biasd = a.to(dev), bw.to(dev), bias.to(dev)
    C = torch.empty((M, N), device=dev, dtype=torch.bfloat16)
    rc = L.bi_gemm_bf16(ad.data_ptr(), K, bd.data_ptr(), bw.shape[1], 1, C.data_ptr(), N, M, N, K, biasd.data_ptr(),
                        torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.equal(C.cpu(), want)
    got = bio.matmul_persistent(ad, bd[:, :N], biasd)
    assert torch.equal(got.cpu(), want)
    assert torch.equal(bio.matmul_persistent(ad[:1], bd[:, :N], biasd), got[:1])
    with bio.set_batch_invariant_mode(True):
        assert torch.equal((ad @ bd[:, :N]).cpu(), O.matmul_single_acc(a, b))


def test_single_accumulator_mm_fp16(dev):
    a = O.gaussian_bf16((300, 1000), 1.0, 0).to(torch.float16)
    w = O.gaussian_bf16((200, 1000), 0.05, 1).to(torch.float16)
    b = O.gaussian_bf16((200,), 1.0, 2).to(torch.float16)
    got = bio.matmul_persistent(a.to(dev), w.to(dev).t(), bias=b.to(dev))
    want = O.matmul_single_acc(a, w.t(), b)
    assert got.dtype == torch.float16
    d = (got.cpu().float() - want.float()).abs()
    assert (d <= 2.0 ** -10 * want.float().abs().clamp_min(2.0 ** -6)).all()   # one fp16 ulp (fp32 order differs)
    for rows in (1, 7, 64):
        assert torch.equal(bio.matmul_persistent(a[:rows].to(dev), w.to(dev).t(), bias=b.to(dev)), got[:rows])
    ai = O.integer_bf16((70, 512), -9, 9, 8).to(torch.float16)
    wi = O.integer_bf16((96, 512), -7, 7, 9).to(torch.float16)
    assert torch.equal(bio.matmul_persistent(ai.to(dev), wi.to(dev).t()).cpu(), O.matmul_single_acc(ai, wi.t()))
    with bio.set_batch_invariant_mode(True):
        assert torch.equal(torch.mm(ai.to(dev), wi.to(dev).t()).cpu(), O.matmul_single_acc(ai, wi.t()))


def test_single_accumulator_mm_fp32(dev):
    g = torch.Generator().manual_seed(4)
    a = torch.randn((130, 1001), generator=g)
    w = torch.randn((77, 1001), generator=g) * 0.05
    b = torch.randn((77,), generator=g)
    got = bio.matmul_persistent(a.to(dev), w.to(dev).t(), bias=b.to(dev))
    want = (a.double() @ w.double().t() + b.double()).float()
    assert got.dtype == torch.float32 and got.shape == (130, 77)
    assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-5 * want.abs().max().item())
    for rows in (1, 7, 64):
        assert torch.equal(bio.matmul_persistent(a[:rows].to(dev), w.to(dev).t(), bias=b.to(dev)), got[:rows])
    ai = O.integer_bf16((70, 512), -9, 9, 8).float()
    wi = O.integer_bf16((96, 512), -7, 7, 9).float()
    with bio.set_batch_invariant_mode(True):
        assert torch.equal(torch.mm(ai.to(dev), wi.to(dev).t()).cpu(), ai @ wi.t())
        assert torch.equal(torch.addmm(b[:1].to(dev).expand(96), ai.to(dev), wi.to(dev).t()).cpu(), ai @ wi.t() + b[0])


def test_silu_mul_parity_and_batch_invariance(dev):
    from llm_reproducibility_amd import ops
    g = torch.Generator().manual_seed(11)
    gu = (torch.randn((300, 2 * 12288), generator=g) * 2).to(torch.bfloat16)
    want = O.silu_mul(gu)
    got = ops.bi_silu_mul(gu.to(dev))
    assert got.shape == want.shape
    assert O.bf16_ulp_distance(got.cpu(), want).max().item() <= 1   # device exp vs host exp: at most one rounding flip
    # gate = 5.9375 is a hard case: silu = 5.92187444, 1.2 fp32 steps below the bf16 boundary 5.921875 -- a quotient
    # that is off by more than one fp32 step lands on the other side
    hard = torch.tensor([[5.9375] * 8 + [-2.375, 0.6171875, 2.4375, -2.34375, 0.1669921875, 7.96875, 1.0, -1.0]], dtype=torch.bfloat16)
    assert torch.equal(ops.bi_silu_mul(hard.to(dev)).cpu(), O.silu_mul(hard))
    for rows in (1, 7, 256):
        assert torch.equal(ops.bi_silu_mul(gu[:rows].to(dev)), got[:rows])
    # a strided view (row stride larger than the row) and a 3-D input
    wide = torch.zeros((16, 2 * 256 + 64), dtype=torch.bfloat16)
    wide[:, :512] = gu[:16, :512]
    assert torch.equal(ops.bi_silu_mul(wide.to(dev)[:, :512]).cpu(), ops.bi_silu_mul(gu[:16, :512].contiguous().to(dev)).cpu())
    assert ops.bi_silu_mul(gu[:12, :64].reshape(3, 4, 64).to(dev)).shape == (3, 4, 32)
    # exact cases: silu(0) * u = 0, silu(40) = 40
    z = torch.zeros((1, 16), dtype=torch.bfloat16)
    z[0, 1] = 40.0
    z[0, 8:] = 2.0
    assert ops.bi_silu_mul(z.to(dev)).cpu().tolist() == [[0.0, 80.0, 0, 0, 0, 0, 0, 0]]


def test_random_shapes_of_the_reductions(dev):
    """Seeded sweep over row counts and widths the fixed-shape tests do not visit (hidden sizes that are not powers of
    two, vocabularies around the 1024-wide pieces, means over inner dimensions): tolerance against fp64 library
    routines or the oracle, and a random row alone reproduces its bits inside the batch."""
    import random
    from llm_reproducibility_amd import ops
    rng = random.Random(3)
    for it in range(30):
        rows = rng.choice([1, 2, 7, 33, 256, 1000])
        hid = rng.choice([64, 128, 136, 1000, 1024, 2560, 5120, 8192])
        print("case", it, rows, hid, flush=True)
        x = O.gaussian_bf16((rows, hid), 1.0, it)
        w = (1 + 0.1 * torch.randn(hid, generator=torch.Generator().manual_seed(it))).to(torch.bfloat16)
        got = bio.rms_norm(x.to(dev), w.to(dev), 1e-6)
        ulp = O.bf16_ulp_distance(got.cpu(), O.rmsnorm(x, w, 1e-6))
        assert ulp.max() <= 2 and (ulp > 0).float().mean() < 0.02, ("rmsnorm", rows, hid)
        r = rng.randrange(rows)
        assert torch.equal(bio.rms_norm(x[r:r + 1].to(dev), w.to(dev), 1e-6), got[r:r + 1]), ("rmsnorm row", rows, hid, r)
        cols = rng.choice([1, 5, 1023, 1024, 1025, 4096, 32000, 50257, 152064])
        rows2 = min(rows, 64)
        lx = 3 * torch.randn((rows2, cols), generator=torch.Generator().manual_seed(100 + it))
        ls = bio.log_softmax(lx.to(dev))
        assert (ls.cpu().double() - torch.log_softmax(lx.double(), -1)).abs().max() < 2e-5, ("log_softmax", rows2, cols)
        r = rng.randrange(rows2)
        assert torch.equal(bio.log_softmax(lx[r:r + 1].to(dev)), ls[r:r + 1]), ("log_softmax row", rows2, cols, r)
        assert (bio.softmax(lx.to(dev)).cpu().double() - torch.softmax(lx.double(), -1)).abs().max() < 1e-6, ("softmax", rows2, cols)
        shp = rng.choice([(rows, 1000), (3, rows, 17), (rows, 5, 64), (2, 3, 4, 5), (rows, 40000)])
        mx = torch.randn(shp, generator=torch.Generator().manual_seed(200 + it))
        d = rng.randrange(len(shp))
        mean = bio.mean_dim(mx.to(dev), d, keepdim=bool(it & 1))
        assert (mean.cpu().double() - mx.double().mean(d, keepdim=bool(it & 1))).abs().max() < 1e-5, ("mean", shp, d)
        inter = rng.choice([8, 64, 1000, 12288])
        gu = O.gaussian_bf16((rows, 2 * inter), 2.0, 300 + it)
        assert O.bf16_ulp_distance(ops.bi_silu_mul(gu.to(dev)).cpu(), O.silu_mul(gu)).max() <= 1, ("silu_mul", rows, inter)


def test_argmax_lowest_index_on_ties(dev):
    from llm_reproducibility_amd import ops
    g = torch.Generator().manual_seed(7)
    for rows, cols in ((1, 151936), (7, 151936), (128, 151936), (3, 5), (4, 1000), (2, 8), (5, 1031)):
        x = torch.randn((rows, cols), generator=g).to(torch.bfloat16)   # bf16 values collide often: many ties
        want = O.argmax_lowest_index(x)
        got = ops.bi_argmax(x.to(dev))
        assert got.dtype == torch.int64 and torch.equal(got.cpu(), want), (rows, cols)
        r = rows - 1
        assert torch.equal(ops.bi_argmax(x[r:r + 1].to(dev)), got[r:r + 1]), "row alone"
    flat = torch.zeros((3, 4096), dtype=torch.bfloat16)
    flat[1, 77] = -0.0
    flat[2] = -1
    flat[2, 4000] = 5
    flat[2, 123] = 5
    assert ops.bi_argmax(flat.to(dev)).tolist() == [0, 0, 123]
    wide = torch.randn((6, 300), generator=g).to(torch.bfloat16).to(dev)
    view = wide[:, 3:203]                                                # strided, 2-byte aligned rows
    assert torch.equal(ops.bi_argmax(view), ops.bi_argmax(view.contiguous()))


def test_argmax_with_step_bookkeeping_equals_argmax_and_the_separate_updates(dev):
    """The token choice that also files the token and advances the sequence state (one launch of a decode step):
    same index as bi_argmax / the oracle on rows full of ties, history written at each row's own count, a full
    history left alone, and every optional argument may be absent."""
    from llm_reproducibility_amd import ops
    g = torch.Generator().manual_seed(11)
    rows, cols, T = 5, 151936, 3
    nxt = torch.full((rows,), -1, dtype=torch.int64, device=dev)
    hist = torch.full((rows, T), -7, dtype=torch.int64, device=dev)
    count = torch.tensor([0, 1, 2, 3, 0], dtype=torch.int64, device=dev)       # row 3: history already full
    pos = torch.tensor([10, 0, 5, 99, 2 ** 40], dtype=torch.int64, device=dev)
    ctx = torch.tensor([11, 1, 6, 100, 7], dtype=torch.int32, device=dev)
    want_hist = hist.clone()
    for stepno in range(2):
        x = torch.randn((rows, cols), generator=g).to(torch.bfloat16)
        want = O.argmax_lowest_index(x)
        c0, p0, l0 = count.clone(), pos.clone(), ctx.clone()
        got = ops.bi_argmax_advance(x.to(dev), nxt, hist, count, pos, ctx)
        assert got is nxt and torch.equal(nxt.cpu(), want) and torch.equal(nxt, ops.bi_argmax(x.to(dev))), stepno
        for r in range(rows):
            if int(c0[r]) < T:
                want_hist[r, int(c0[r])] = want[r]
        assert torch.equal(hist, want_hist), stepno
        assert torch.equal(count, c0 + 1) and torch.equal(pos, p0 + 1) and torch.equal(ctx, l0 + 1), stepno
    # nothing but the token
    x = torch.randn((2, 1000), generator=g).to(torch.bfloat16)
    two = torch.empty(2, dtype=torch.int64, device=dev)
    assert torch.equal(ops.bi_argmax_advance(x.to(dev), two).cpu(), O.argmax_lowest_index(x))
    # positions only; and a history without its count is refused
    p1 = torch.zeros(2, dtype=torch.int64, device=dev)
    ops.bi_argmax_advance(x.to(dev), two, positions=p1)
    assert p1.tolist() == [1, 1]
    with pytest.raises(ValueError):
        ops.bi_argmax_advance(x.to(dev), two, history=torch.zeros((2, 4), dtype=torch.int64, device=dev))
    with pytest.raises(ValueError):
        ops.bi_argmax_advance(x.to(dev), two, ctx_len=torch.zeros(2, dtype=torch.int64, device=dev))   # int32 required


def test_aten_overrides_route_to_the_hip_kernels(dev):
    a = O.gaussian_bf16((20, 512), 1.0, 0).to(dev)
    w = O.gaussian_bf16((64, 512), 0.1, 1).to(dev)
    b = O.gaussian_bf16((64,), 1.0, 2).to(dev)
    logits = torch.randn((5, 3000), device=dev)
    with bio.set_batch_invariant_mode(True):
        assert bio.is_batch_invariant_mode_enabled()
        assert torch.equal(torch.mm(a, w.t()), bio.matmul_persistent(a, w.t()))
        assert torch.equal(torch.nn.functional.linear(a, w, b), bio.matmul_persistent(a, w.t(), b))
        assert torch.equal(torch.log_softmax(logits, -1), bio.log_softmax(logits))
        assert torch.equal(torch.softmax(logits, -1), bio.softmax(logits))
        assert torch.equal(logits.mean(-1, keepdim=True), bio.mean_dim(logits, -1, keepdim=True))
        m2 = logits.reshape(5, 30, 100).mean(dim=(1, 2))
        assert (m2 - logits.mean(-1)).abs().max() < 1e-6
    assert not bio.is_batch_invariant_mode_enabled()
    ref = torch.log_softmax(logits, -1)              # stock kernel again after leaving the mode
    assert (ref - bio.log_softmax(logits)).abs().max() < 1e-5


def test_empty_inputs_are_handled_without_a_launch(dev):
    from llm_reproducibility_amd import ops
    from llm_reproducibility_amd.tbik import matmul_tp_persistent, tree_combine
    w = O.gaussian_bf16((64, 512), 0.1, 1).to(dev)
    e = torch.empty((0, 512), dtype=torch.bfloat16, device=dev)
    assert matmul_tp_persistent(e, w.t()).shape == (0, 64)
    assert bio.matmul_persistent(e, w.t()).shape == (0, 64)
    assert bio.rms_norm(e, torch.ones(512, dtype=torch.bfloat16, device=dev), 1e-6).shape == (0, 512)
    assert bio.log_softmax(torch.empty((0, 100), device=dev)).shape == (0, 100)
    assert bio.mean_dim(torch.empty((0, 16), device=dev), -1).shape == (0,)
    assert ops.bi_silu_mul(torch.empty((0, 64), dtype=torch.bfloat16, device=dev)).shape == (0, 32)
    z = torch.empty((0, 8), dtype=torch.bfloat16, device=dev)
    assert tree_combine([z, z]).shape == (0, 8)
    torch.cuda.synchronize()
