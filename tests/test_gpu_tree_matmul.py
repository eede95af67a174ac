"""GPU parity of the tree-ordered matmul (tbik_gemm_bf16 through the C ABI) against the CPU oracle.

Bit-exact on integer-valued inputs (every leaf sum exact, so only the tree order and the rounding
decide the result); on Gaussian inputs each element must be within 1 bf16 ulp of the oracle OR within
2^-8 of the output scale; invariance across simulated TP = 1/2/4/8 and across batch sizes is bitwise.
"""
import os

import numpy as np
import pytest
import torch

from oracle import tbik_oracle as O
from llm_reproducibility_amd.tbik import choose_leaf_k, matmul_tp_persistent, tree_combine

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kat_tree_matmul.npz")


def bits(t):
    return t.contiguous().view(torch.int16)


def assert_bitwise(a, b, msg=""):
    a, b = a.cpu(), b.cpu()
    if not torch.equal(bits(a), bits(b)):
        d = (a.float() - b.float()).abs()
        raise AssertionError(f"{msg}: {int((bits(a) != bits(b)).sum())} of {a.numel()} elements differ, max |diff| {d.max().item()}")


def assert_close_to_oracle(got, want, msg=""):
    """<= 1 bf16 ulp, or |diff| <= 2^-8 * max|want| (the tolerance the contract states for random inputs)."""
    got, want = got.cpu(), want.cpu()
    ulp = O.bf16_ulp_distance(got, want)
    diff = (got.float() - want.float()).abs()
    scale = want.float().abs().max().item()
    bad = (ulp > 1) & (diff > 2.0 ** -8 * scale)
    assert not bad.any(), f"{msg}: {int(bad.sum())} elements off; max ulp {int(ulp.max())}, max diff {diff.max().item()}, scale {scale}"


def sim_tp(A, W_kn, p, leaf_k):
    K = A.shape[1]
    ks = K // p
    parts = [matmul_tp_persistent(A[:, r * ks:(r + 1) * ks], W_kn[r * ks:(r + 1) * ks, :], leaf_k=leaf_k) for r in range(p)]
    return parts[0] if p == 1 else tree_combine(parts)


def test_rational_known_answers(dev):
    z = np.load(GOLDEN)
    for n in sorted({k[:-2] for k in z.files if k.endswith("_A")}):
        A = torch.from_numpy(z[n + "_A"].astype(np.float32)).to(torch.bfloat16).to(dev)
        B = torch.from_numpy(z[n + "_B"].astype(np.float32)).to(torch.bfloat16).to(dev)
        C = torch.from_numpy(z[n + "_C"].view(np.int16).copy()).view(torch.bfloat16)
        leaf = int(z[n + "_leaf"])
        print("case", n, tuple(A.shape), tuple(B.shape), leaf, flush=True)
        assert_bitwise(matmul_tp_persistent(A, B, leaf_k=leaf), C, n)
        # the weight as nn.Linear stores it ([N,K], handed over as weight.t())
        Wnk = B.t().contiguous()
        assert_bitwise(matmul_tp_persistent(A, Wnk.t(), leaf_k=leaf), C, n + " (weight.t())")


# (M, N, K, leaf): tails in M and N, every tile configuration, FLB in {1,2,3,5,25}, 0..5 binary levels
INT_SHAPES = [
    (1, 64, 256, 256), (3, 72, 512, 256), (16, 128, 768, 256), (17, 200, 1536, 256), (64, 136, 2048, 256),
    (65, 128, 1280, 256), (130, 264, 3072, 256), (257, 512, 4096, 256), (128, 128, 12288, 256),
    (33, 96, 3200, 128), (129, 160, 6400, 128), (20, 64, 6400, 256), (8, 24, 8192, 256), (300, 4, 512, 256),
]


@pytest.mark.parametrize("M,N,K,leaf", INT_SHAPES)
def test_integer_inputs_match_oracle_bitwise(dev, M, N, K, leaf):
    print("case", M, N, K, leaf, flush=True)
    A = O.integer_bf16((M, K), -9, 9, 10 + M)
    B = O.integer_bf16((K, N), -7, 7, 20 + N)
    want = O.matmul_tree(A, B, leaf=leaf)
    Wnk = B.t().contiguous().to(dev)
    got = matmul_tp_persistent(A.to(dev), Wnk.t(), leaf_k=leaf)
    assert got.shape == (M, N) and got.dtype == torch.bfloat16 and got.is_contiguous()
    assert_bitwise(got, want, f"{M}x{N}x{K}")


# (M, N, K, leaf): grids of 128x256 tiles.  Both large-M kernels (one binary level in registers / two, the latter for
# groups of two leaves from two levels on and for any tree from four levels on), with and without a K split in front,
# leaves of 256 and 128, ragged tiles in M and N
LARGE_TILE_SHAPES = [
    (1000, 4000, 8192, 256), (520, 2100, 12288, 256), (1024, 2048, 6400, 128), (2048, 2048, 2048, 256),
    (300, 5000, 4096, 256), (640, 1024, 16384, 256),
]


@pytest.mark.parametrize("M,N,K,leaf", LARGE_TILE_SHAPES)
def test_large_tile_kernels_match_oracle_bitwise(dev, M, N, K, leaf):
    print("case", M, N, K, leaf, flush=True)
    A_wide = O.integer_bf16((M, K + 8), -9, 9, 50 + M % 89)
    A = A_wide[:, 8:]                       # a strided view (row stride K + 8)
    Wnk = O.integer_bf16((N, K), -7, 7, 60 + N % 97)
    bias = O.integer_bf16((N,), -300, 300, 6)
    Ad, Wd = A_wide.to(dev)[:, 8:], Wnk.to(dev)
    assert_bitwise(matmul_tp_persistent(Ad, Wd.t(), leaf_k=leaf), O.matmul_tree(A, Wnk.t(), leaf=leaf), f"{M}x{N}x{K}")
    assert_bitwise(matmul_tp_persistent(Ad, Wd.t(), bias.to(dev), leaf_k=leaf), O.matmul_tree(A, Wnk.t(), bias, leaf=leaf), "bias")
    # fp16 operands on the same grids (the first of the two kernels, instantiated for fp16)
    h = matmul_tp_persistent(Ad.to(torch.float16), Wd.to(torch.float16).t(), bias.to(dev).to(torch.float16), leaf_k=leaf)
    assert_bitwise(h, O.matmul_tree(A.to(torch.float16), Wnk.to(torch.float16).t(), bias.to(torch.float16), leaf=leaf), "fp16")


# grids that do not fill whole rounds of work-groups: the dispatcher cuts the columns into two regions, each with a K split
# of its own, and launches both at once (o_proj 32B at 512 and 1024 rows: 4 and 16 shards / 2 and 8; a leaf-128 tree;
# a region that is not cut at all next to one cut in two)
@pytest.mark.parametrize("M,N,K,leaf", [(512, 5120, 8192, 256), (1024, 5120, 8192, 256), (2048, 5120, 6400, 128), (2048, 5120, 2048, 256), (1024, 5120, 16384, 256)])
def test_column_regions_with_their_own_k_split_match_oracle_bitwise(dev, M, N, K, leaf):
    print("case", M, N, K, leaf, flush=True)
    A = O.integer_bf16((M, K), -9, 9, 70 + M % 89)
    Wnk = O.integer_bf16((N, K), -7, 7, 80 + N % 97)
    bias = O.integer_bf16((N,), -300, 300, 7)
    Ad, Wd, bd = A.to(dev), Wnk.to(dev), bias.to(dev)
    got = matmul_tp_persistent(Ad, Wd.t(), bd, leaf_k=leaf)
    assert_bitwise(got, O.matmul_tree(A, Wnk.t(), bias, leaf=leaf), f"{M}x{N}x{K}")
    # any block of columns computed alone (another plan, other regions) has the same bits
    for lo, hi in ((0, 256), (256, 1280), (4096, N), (1000, 3000)):
        part = matmul_tp_persistent(Ad, Wd[lo:hi].t(), bd[lo:hi], leaf_k=leaf)
        assert torch.equal(part, got[:, lo:hi]), (lo, hi)
    # Gaussian operands: rows alone and simulated TP agree bitwise with the batch
    g = O.gaussian_bf16((M, K), 1.0, 71).to(dev)
    gw = O.gaussian_bf16((N, K), 0.02, 72).to(dev)
    full = matmul_tp_persistent(g, gw.t(), leaf_k=leaf)
    assert torch.equal(matmul_tp_persistent(g[:1], gw.t(), leaf_k=leaf), full[:1])
    assert torch.equal(matmul_tp_persistent(g[M - 70:], gw.t(), leaf_k=leaf), full[M - 70:])
    assert torch.equal(sim_tp(g, gw.t(), 2, leaf), full)
    if M == 512:  # the same grid in fp16 (the first of the two kernels, instantiated for fp16)
        h = matmul_tp_persistent(Ad.to(torch.float16), Wd.to(torch.float16).t(), bd.to(torch.float16), leaf_k=leaf)
        assert_bitwise(h, O.matmul_tree(A.to(torch.float16), Wnk.to(torch.float16).t(), bias.to(torch.float16), leaf=leaf), "fp16")


# 64..512 rows with short K shards take 128x128 tiles with the shard's tree in registers: shards of one group of 2, 3 or
# 5 leaves, shards of two groups (one binary level inside the shard), a ragged last tile, a width that is not a multiple
# of 4 (element-wise stores of the partial results), 160..256 work-groups
@pytest.mark.parametrize("M,N,K", [(128, 4096, 4096), (100, 3072, 6144), (128, 4000, 12288), (96, 2048, 8192),
                                   (128, 7162, 5120), (128, 4096, 8192), (113, 5120, 2048), (64, 4096, 6144), (80, 2048, 12288), (256, 4096, 4096), (192, 2048, 6144),
                                   (160, 1500, 8192), (500, 1024, 6144)])
def test_narrow_tiles_for_short_shards_match_oracle_and_the_other_kernels_bitwise(dev, M, N, K):
    print("case", M, N, K, flush=True)
    A = O.integer_bf16((M, K), -9, 9, 170 + M % 89)
    Wnk = O.integer_bf16((N, K), -7, 7, 180 + N % 97)
    bias = O.integer_bf16((N,), -300, 300, 9)
    Ad, Wd, bd = A.to(dev), Wnk.to(dev), bias.to(dev)
    got = matmul_tp_persistent(Ad, Wd.t(), bd, leaf_k=256)
    assert_bitwise(got, O.matmul_tree(A, Wnk.t(), bias, leaf=256), f"{M}x{N}x{K} with bias")
    assert_bitwise(matmul_tp_persistent(Ad, Wd.t(), leaf_k=256), O.matmul_tree(A, Wnk.t(), leaf=256), f"{M}x{N}x{K}")
    # Gaussian operands: fewer rows (the few-rows kernels), more rows (128x256 tiles), a block of columns and the
    # simulated TP shards all run on other kernels and agree bitwise with this batch (how close those bits are to the
    # oracle's on Gaussian data is the subject of test_gaussian_inputs_within_one_ulp_of_oracle)
    g = O.gaussian_bf16((M + 172, K), 1.0, 171).to(dev)
    gw = O.gaussian_bf16((N, K), 0.02, 172).to(dev)
    full = matmul_tp_persistent(g[:M], gw.t(), leaf_k=256)
    assert torch.equal(matmul_tp_persistent(g[:1], gw.t(), leaf_k=256), full[:1])
    assert torch.equal(matmul_tp_persistent(g[M - 40:M], gw.t(), leaf_k=256), full[M - 40:])
    assert torch.equal(matmul_tp_persistent(g, gw.t(), leaf_k=256)[:M], full)
    assert torch.equal(matmul_tp_persistent(g[:M], gw[256:1024].t(), leaf_k=256), full[:, 256:1024])
    groups = K // 256 // O.tree_params(K, 256)[1]  # a TP degree has to cut K into aligned subtrees
    for p in (2, 4, 8):
        if groups % p == 0:
            assert torch.equal(sim_tp(g[:M], gw.t(), p, 256), full), p


def test_large_tile_kernels_seeded_sweep_of_random_shapes(dev):
    """Random grids of 128x256 tiles (64 or more rows, ragged edges, trees of every depth and group size the leaf count
    allows, leaves of 128 and 256, bf16 and fp16, with and without bias): bit-exact against the oracle on integer inputs."""
    import random
    rng = random.Random(2024)
    for it in range(14):
        leaf = rng.choice([256, 256, 256, 128])
        T = rng.choice([2, 3, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 64, 96])
        M = rng.choice([64, 100, 128, 200, 333, 512, 777, 1024, 1500])
        N = rng.choice([256, 520, 1000, 1536, 2048, 3000, 4096, 5120])
        K = leaf * T
        if M * N * K > 1.2e11:
            N = 1024
        f16 = rng.random() < 0.3
        use_bias = rng.random() < 0.5
        print("case", it, M, N, K, leaf, "fp16" if f16 else "bf16", "bias" if use_bias else "", flush=True)
        A = O.integer_bf16((M, K), -9, 9, 100 + it)
        Wnk = O.integer_bf16((N, K), -3, 3, 200 + it)
        bias = O.integer_bf16((N,), -64, 64, 300 + it) if use_bias else None
        if f16:
            A, Wnk, bias = A.to(torch.float16), Wnk.to(torch.float16), (bias.to(torch.float16) if use_bias else None)
        want = O.matmul_tree(A, Wnk.t(), bias, leaf=leaf)
        got = matmul_tp_persistent(A.to(dev), Wnk.to(dev).t(), bias.to(dev) if use_bias else None, leaf_k=leaf)
        assert_bitwise(got, want, f"case {it}: {M}x{N}x{K} leaf {leaf}")


# (M, N, K, leaf): a few rows (up to 16 when the tree has at most four aligned subtrees) and a grid of 16-column strips that loads every CU alike: the one-launch kernel that
# cuts K over the waves of a work-group (2/4/8 waves, FLB in {1,2,3,5,25}, up to three binary levels inside a wave,
# a ragged last strip)
STRIP_SHAPES = [
    (1, 4096, 512, 256), (3, 2056, 1024, 256), (4, 1024, 2048, 256), (2, 3000, 4096, 256), (4, 1040, 6144, 256),
    (2, 4090, 12288, 256), (1, 8192, 4096, 256), (3, 1024, 16384, 256), (4, 1040, 8192, 128), (1, 4096, 25600, 128),
    (2, 4096, 1280, 128), (8, 2560, 9728, 256), (16, 1024, 1536, 256), (13, 4096, 2560, 128),
]


@pytest.mark.parametrize("M,N,K,leaf", STRIP_SHAPES)
def test_few_rows_one_launch_kernel_matches_oracle_bitwise(dev, M, N, K, leaf):
    print("case", M, N, K, leaf, flush=True)
    A_wide = O.integer_bf16((M, K + 8), -9, 9, 30 + M)
    A = A_wide[:, 8:]                       # a strided view (row stride K + 8)
    Wnk = O.integer_bf16((N, K), -7, 7, 40 + N % 97)
    bias = O.integer_bf16((N,), -300, 300, 5)
    want = O.matmul_tree(A, Wnk.t(), leaf=leaf)
    Ad, Wd = A_wide.to(dev)[:, 8:], Wnk.to(dev)
    got = matmul_tp_persistent(Ad, Wd.t(), leaf_k=leaf)
    assert got.shape == (M, N) and got.is_contiguous()
    assert_bitwise(got, want, f"{M}x{N}x{K}")
    assert_bitwise(matmul_tp_persistent(Ad, Wd.t(), bias.to(dev), leaf_k=leaf), O.matmul_tree(A, Wnk.t(), bias, leaf=leaf), "bias")
    # the same rows inside a batch of 40 go through another kernel: same bits
    big = torch.cat([Ad, O.integer_bf16((40 - M, K), -9, 9, 77).to(dev)])
    assert_bitwise(matmul_tp_persistent(big, Wd.t(), leaf_k=leaf)[:M], want, "rows inside a larger batch")
    if leaf == 256:
        h = matmul_tp_persistent(Ad.to(torch.float16), Wd.to(torch.float16).t(), leaf_k=leaf)
        assert_bitwise(h, O.matmul_tree(A.to(torch.float16), Wnk.to(torch.float16).t(), leaf=leaf), "fp16")


@pytest.mark.parametrize("M,N,K", [(2, 4096, 4096), (16, 1024, 3072), (96, 512, 4096), (300, 1024, 12288), (256, 4096, 2048)])
def test_c_abi_writes_into_a_strided_and_a_misaligned_output(dev, M, N, K):
    """The entry point itself (no wrapper): C is a column block of a wider matrix (ldc > N), then the same block
    shifted by one element (2-byte aligned only, scalar stores); every kernel family and the K-cut path."""
    from llm_reproducibility_amd import _lib
    L = _lib.lib()
    print("case", M, N, K, flush=True)
    A = O.integer_bf16((M, K), -9, 9, 3).to(dev)
    W = O.integer_bf16((N, K), -7, 7, 4).to(dev)
    bias = O.integer_bf16((N,), -300, 300, 5).to(dev)
    want = matmul_tp_persistent(A, W.t(), bias)
    nws = L.tbik_gemm_workspace_bytes(M, N, K, 256)
    ws = torch.empty(max(nws, 1), device=dev, dtype=torch.uint8)
    stream = torch.cuda.current_stream().cuda_stream
    for shift in (8, 9):
        wide = torch.full((M, N + 24), 7.0, device=dev, dtype=torch.bfloat16)
        cptr = wide.data_ptr() + 2 * shift
        rc = L.tbik_gemm_bf16(A.data_ptr(), K, W.data_ptr(), 1, K, cptr, N + 24, M, N, K, 256, bias.data_ptr(),
                              ws.data_ptr() if nws else None, nws, stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        assert_bitwise(wide[:, shift:shift + N], want, f"shift {shift}")
        assert bool((wide[:, :shift] == 7).all()) and bool((wide[:, shift + N:] == 7).all()), "wrote outside its block"


def test_bias_strided_a_and_row_major_b(dev):
    M, N, K = 70, 96, 1536
    A_wide = O.integer_bf16((M, 2 * K), -9, 9, 1)
    B = O.integer_bf16((K, N), -7, 7, 2)
    bias = O.integer_bf16((N,), -300, 300, 3)
    A = A_wide[:, K:]                      # row stride 2K, offset K: a shard's view of a wider activation
    want = O.matmul_tree(A, B, bias)
    Ad = A_wide.to(dev)[:, K:]
    assert not Ad.is_contiguous()
    got = matmul_tp_persistent(Ad, B.to(dev), bias.to(dev))     # row-major [K,N] operand
    assert_bitwise(got, want, "bias + strided A + row-major B")
    odd = A_wide.to(dev)[:, 3:3 + K]       # misaligned view: repacked by the wrapper, same bits
    assert_bitwise(matmul_tp_persistent(odd, B.to(dev)), O.matmul_tree(A_wide[:, 3:3 + K], B), "misaligned A")


# (M, N, K, leaf): row-major B[K,N] consumed in place -- both tile shapes, column tails that cut an 8-wide block
# (N = 100, 1001 elements... with a row stride that is a multiple of 8), the K-cut path, leaf 128, deep trees
ROWMAJOR_SHAPES = [(1, 64, 512, 256), (16, 104, 768, 256), (17, 200, 1536, 256), (70, 136, 2048, 256), (300, 1000, 1024, 256),
                   (33, 96, 3200, 128), (8, 24, 8192, 256), (130, 4096, 12288, 256), (64, 72, 6400, 128)]


@pytest.mark.parametrize("M,N,K,leaf", ROWMAJOR_SHAPES)
def test_row_major_b_is_consumed_in_place_bitwise(dev, M, N, K, leaf):
    """The C ABI with ldb_n == 1 (B[K,N], N contiguous, the layout of simple_matmul.py): no repack anywhere -- the raw
    entry point is called on the row-major buffer -- and the bits equal the oracle's and the [N,K] path's."""
    from llm_reproducibility_amd import _lib
    L = _lib.lib()
    print("case", M, N, K, leaf, flush=True)
    A = O.integer_bf16((M, K), -9, 9, 50 + M)
    ldb = N + (-N) % 8 + 8                                   # row stride: a multiple of 8, wider than N
    Bw = O.integer_bf16((K, ldb), -7, 7, 60 + N % 89)
    B = Bw[:, :N]
    bias = O.integer_bf16((N,), -300, 300, 7)
    want = O.matmul_tree(A, B, bias, leaf=leaf)
    Ad, Bd, bd = A.to(dev), Bw.to(dev), bias.to(dev)
    nws = L.tbik_gemm_workspace_bytes_rowmajor_b(M, N, K, leaf, 0)
    ws = torch.empty(max(nws, 1), device=dev, dtype=torch.uint8)
    C = torch.empty((M, N), device=dev, dtype=torch.bfloat16)
    rc = L.tbik_gemm_bf16(Ad.data_ptr(), K, Bd.data_ptr(), ldb, 1, C.data_ptr(), N, M, N, K, leaf, bd.data_ptr(),
                          ws.data_ptr() if nws else None, nws, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert_bitwise(C, want, "row-major B through the C ABI")
    # the wrapper hands a row-major view over as it is (same bits as the [N,K] form, which runs other kernels)
    got = matmul_tp_persistent(Ad, Bd[:, :N], bd, leaf_k=leaf)
    assert_bitwise(got, want, "row-major B through the wrapper")
    assert_bitwise(matmul_tp_persistent(Ad, Bd[:, :N].t().contiguous().t(), bd, leaf_k=leaf), want, "[N,K] form")
    if leaf == 256 and M <= 70:
        h = matmul_tp_persistent(Ad.to(torch.float16), Bd[:, :N].to(torch.float16), leaf_k=leaf)
        assert_bitwise(h, O.matmul_tree(A.to(torch.float16), B.to(torch.float16), leaf=leaf), "fp16, row-major B")


def test_row_major_b_simulated_tp_as_the_reference_script_runs_it(dev):
    """simple_matmul.py:23-43 on its own layout: A[M,K] and B[K,N] both row-major, K cut into shards by slicing rows of
    B (still row-major views), shard outputs combined in the tree: bitwise equal to the unsplit product."""
    M, K, N = 96, 6144, 520
    A = O.gaussian_bf16((M, K), 1.0, 0).to(dev)
    B = O.gaussian_bf16((K, N), 1.0, 1).to(dev)
    full = matmul_tp_persistent(A, B)
    for p in (2, 4, 8):
        assert_bitwise(sim_tp(A, B, p, 256), full, f"TP={p}")
    assert_bitwise(matmul_tp_persistent(A[:7], B), full[:7], "batch prefix")
    assert_close_to_oracle(full, O.matmul_tree(A.cpu(), B.cpu()), "row-major B, Gaussian")


def test_row_major_b_repacked_from_many_rows_on_gives_the_same_bits(dev):
    """From 1024 rows on (2048 for the single-accumulator mm) the wrappers repack a row-major [K,N] operand into the
    native layout, because the in-place path runs on the small tiles only; on either side of the switch the bits are
    those of the [N,K] form."""
    from llm_reproducibility_amd import ops
    from llm_reproducibility_amd.bio import batch_invariant_ops as bio
    K, N = 2048, 1536
    B = O.gaussian_bf16((K, N), 0.02, 3).to(dev)                 # row-major [K,N]
    Wt = B.t().contiguous().t()                                  # the same matrix as an [N,K] weight, transposed view
    assert B.stride(1) == 1 and Wt.stride(0) == 1
    for M in (ops._REPACK_ROWS_TREE - 1, ops._REPACK_ROWS_TREE, ops._REPACK_ROWS_MM - 1, ops._REPACK_ROWS_MM):
        print("case row-major B rows", M, flush=True)
        A = O.gaussian_bf16((M, K), 1.0, M).to(dev)
        assert_bitwise(matmul_tp_persistent(A, B), matmul_tp_persistent(A, Wt), f"tree matmul, {M} rows")
        assert torch.equal(bio.matmul_persistent(A, B), bio.matmul_persistent(A, Wt)), M
    assert ops._weight_operand(B, ops._REPACK_ROWS_TREE - 1, True)[1] != 1      # in place
    assert ops._weight_operand(B, ops._REPACK_ROWS_TREE, True)[1:] == (1, K)    # repacked: [N,K], K contiguous
    assert ops._weight_operand(B, ops._REPACK_ROWS_MM - 1, False)[1] != 1
    assert ops._weight_operand(B, ops._REPACK_ROWS_MM, False)[1:] == (1, K)


@pytest.mark.parametrize("M,N,K", [(256, 4096, 4096), (128, 512, 12288), (16, 256, 12288), (1, 128, 8192)])
def test_gaussian_inputs_within_one_ulp_of_oracle(dev, M, N, K):
    print("case", M, N, K, flush=True)
    A = O.gaussian_bf16((M, K), 1.0, 0) if K != 12288 else O.silu_gated_bf16((M, K), 0)
    Wnk = O.gaussian_bf16((N, K), 0.02, 1)
    want = O.matmul_tree(A, Wnk.t())
    got = matmul_tp_persistent(A.to(dev), Wnk.to(dev).t())
    assert_close_to_oracle(got, want, f"{M}x{N}x{K}")
    for p in (2, 4, 8):
        assert_bitwise(sim_tp(A.to(dev), Wnk.to(dev).t(), p, 256), got, f"TP={p}")


def _invariance(dev, K, N, Ms, x_kind, max_m):
    leaf = choose_leaf_k(K)
    X = (O.silu_gated_bf16((max_m, K), 0) if x_kind == "silu" else O.gaussian_bf16((max_m, K), 1.0, 0)).to(dev)
    Wt = O.gaussian_bf16((N, K), 0.02, 1).to(dev).t()
    full = matmul_tp_persistent(X, Wt, leaf_k=leaf)
    for p in (2, 4, 8):
        print("case K", K, "TP", p, flush=True)
        assert_bitwise(sim_tp(X, Wt, p, leaf), full, f"K={K} TP={p} M={max_m}")
    for M in Ms:
        print("case K", K, "M", M, flush=True)
        sub = matmul_tp_persistent(X[:M], Wt, leaf_k=leaf)
        assert_bitwise(sub, full[:M], f"K={K} batch prefix M={M}")
        for p in (2, 8):
            assert_bitwise(sim_tp(X[:M], Wt, p, leaf), full[:M], f"K={K} TP={p} M={M}")
    # a row computed alone equals the same row inside the batch (row 777 of the large batch)
    i = min(777, max_m - 1)
    assert_bitwise(matmul_tp_persistent(X[i:i + 1], Wt, leaf_k=leaf), full[i:i + 1], f"K={K} row {i} alone")
    torch.cuda.synchronize()


def test_invariance_qwen3_8b_down_proj(dev):
    _invariance(dev, 12288, 4096, (1, 16, 128), "silu", 2048)


def test_headline_shape_matches_the_oracle_at_full_size(dev):
    """M=2048, K=12288, N=4096 (the benchmark's workload, every parked tree level of the large-M kernel in use)
    against the CPU oracle on the same seeded inputs: each element within 1 bf16 ulp of the oracle OR within 2^-8 of
    the output scale (the stated tolerance for random inputs: the fp32 order inside a leaf is hardware defined), and
    on integer-valued inputs of the same shape bit for bit."""
    M, K, N = 2048, 12288, 4096
    X = O.silu_gated_bf16((M, K), 0)
    Wnk = O.gaussian_bf16((N, K), 0.02, 1)
    print("case headline gaussian", flush=True)
    want = O.matmul_tree(X, Wnk.t())
    got = matmul_tp_persistent(X.to(dev), Wnk.to(dev).t()).cpu()
    assert_close_to_oracle(got, want, "headline")
    ulp = O.bf16_ulp_distance(got, want)
    # the rounding of a leaf flips at most one bf16 step where the fp32 orders differ: the bulk is bit-equal
    assert float((ulp == 0).float().mean()) > 0.9, float((ulp == 0).float().mean())
    print("case headline integer", flush=True)
    Xi = O.integer_bf16((M, K), -9, 9, 5)
    Wi = O.integer_bf16((N, K), -7, 7, 6)
    assert_bitwise(matmul_tp_persistent(Xi.to(dev), Wi.to(dev).t()), O.matmul_tree(Xi, Wi.t()), "headline, integer inputs")


@pytest.mark.parametrize("name,M,K,N,leaf", [
    ("o_proj 32B", 4096, 8192, 5120, 256),
    ("down_proj 32B", 4096, 25600, 5120, 128),
    ("down_proj 32B mid-sized batch", 512, 25600, 5120, 128),
])
def test_qwen3_32b_shapes_match_the_oracle_bit_for_bit_at_full_size(dev, name, M, K, N, leaf):
    """The row-split layers of the 32B configuration at their full sizes on integer-valued inputs (every leaf sum an
    exact integer in fp32 whatever the order inside the leaf, so only the tree order and the bf16 roundings decide the
    bits): K = 8192 is a tree of 32 leaves in groups of two, K = 25600 with leaves of 128 a tree of 200 leaves in
    groups of 25 under three binary levels (src/tbik/tree_based_matmul.py:242-249 with the leaf of the layer)."""
    assert O.tree_params(K, leaf)[1:] == ((2, 5) if K == 8192 else (25, 4))
    Xi = O.integer_bf16((M, K), -9, 9, 15)
    Wi = O.integer_bf16((N, K), -7, 7, 16)
    print("case", name, M, K, N, leaf, flush=True)
    got = matmul_tp_persistent(Xi.to(dev), Wi.to(dev).t(), leaf_k=leaf).cpu()
    want = O.matmul_tree(Xi, Wi.t(), leaf=leaf)
    assert_bitwise(got, want, name)
    assert want.float().abs().max() > 2048          # sums far beyond the 8 significant bits: the roundings matter


def _plan_signatures():
    """One small representative shape per distinct decision of the dispatcher over a sweep: (path, K splits, one or two
    launches for column regions, leaf, class of row count) -> (M, N, K)."""
    import ctypes
    import itertools
    from llm_reproducibility_amd import _lib
    L = _lib.lib()
    out = (ctypes.c_int * 5)()
    Ms = (1, 2, 4, 8, 16, 17, 48, 64, 96, 128, 160, 256, 384, 512, 768, 1024, 2048, 4096)
    Ns = (256, 512, 1024, 1536, 2048, 3072, 4096, 5120, 6144, 8192)
    Ks = ((512, 256), (1024, 256), (1536, 256), (2048, 256), (3072, 256), (4096, 256), (6144, 256), (8192, 256), (12288, 256),
          (16384, 256), (1280, 128), (3200, 128), (6400, 128), (25600, 128))
    best = {}
    for M, N, (K, leaf) in itertools.product(Ms, Ns, Ks):
        assert L.tbik_gemm_plan_info(M, N, K, leaf, 0, 0, out) == 0
        sig = (out[0], out[1], out[3], out[4], leaf, (M > 16) + (M > 64) + (M > 128) + (M > 512))
        if sig not in best or M * N * K < best[sig][0] * best[sig][1] * best[sig][2]:
            best[sig] = (M, N, K)
    return best


def test_every_decision_of_the_dispatcher_over_a_sweep_gives_the_same_bits(dev):
    """Which kernel, which K split and which column regions serve a shape comes from measured thresholds; a threshold
    that sends a shape to a pairing nobody tried must not change a bit.  For one representative of every distinct decision
    in a sweep of 2520 shapes (all four paths, K cut into 1 .. 32, regions in one and in two launches, both leaf sizes):
    the product equals the same product computed in column chunks of 128 and row chunks of 16 -- small problems that
    take other paths -- bit for bit, and, where the CPU oracle is quick, the oracle on integer inputs."""
    sigs = _plan_signatures()
    assert {s[0] for s in sigs} == {0, 1, 2, 3} and len(sigs) >= 60
    for sig, (M, N, K) in sorted(sigs.items()):
        leaf = sig[4]
        print("case plan", sig, "shape", M, N, K, flush=True)
        A = O.gaussian_bf16((M, K), 1.0, M + K).to(dev)
        Wt = O.gaussian_bf16((N, K), 0.02, N).to(dev).t()
        got = matmul_tp_persistent(A, Wt, leaf_k=leaf)
        ref = torch.empty_like(got)
        for n0 in range(0, N, 128):                      # every element again, as part of a much smaller problem
            for m0 in range(0, M, 16 if M <= 64 else 1024):
                m1 = min(M, m0 + (16 if M <= 64 else 1024))
                ref[m0:m1, n0:n0 + 128] = matmul_tp_persistent(A[m0:m1], Wt[:, n0:n0 + 128], leaf_k=leaf)
        assert_bitwise(got, ref, f"plan {sig} on {M}x{N}x{K}")
        if M * N * K <= 2e9:
            Ai, Wi = O.integer_bf16((M, K), -9, 9, 1), O.integer_bf16((N, K), -7, 7, 2)
            assert_bitwise(matmul_tp_persistent(Ai.to(dev), Wi.to(dev).t(), leaf_k=leaf), O.matmul_tree(Ai, Wi.t(), leaf=leaf),
                           f"plan {sig} against the oracle")


def test_invariance_qwen3_32b_o_proj(dev):
    _invariance(dev, 8192, 5120, (1, 64, 512), "gauss", 4096)


def test_invariance_qwen3_32b_down_proj_leaf128(dev):
    # 25600 / 8 = 3200 is not a multiple of 256: the layer uses leaf 128 at EVERY TP degree
    assert choose_leaf_k(25600) == 128
    _invariance(dev, 25600, 5120, (1, 64, 512), "gauss", 4096)


def test_invariance_with_k_cut_into_32_subtrees(dev):
    # 32 leaves and few column tiles: the small batches are cut into 16 and 32 one-leaf shards, the large one is not
    _invariance(dev, 8192, 2048, (64, 128, 200), "gauss", 1024)
    _invariance(dev, 4096, 1024, (100,), "gauss", 512)


def test_random_shapes_tp_batch_and_row_invariance(dev):
    """Seeded sweep over (leaf, leaves, M, N): every legal simulated TP split, a random batch prefix and a random single
    row reproduce the bits of the full call, whichever kernels the dispatcher picks for the pieces."""
    import random
    rng = random.Random(5)
    for it in range(40):
        leaf = rng.choice([256, 256, 128])
        T = rng.choice([2, 4, 6, 8, 12, 16, 24, 32, 40, 48, 64])
        M = rng.choice([1, 3, 4, 5, 16, 17, 64, 65, 128, 200, 300, 600])
        N = rng.choice([64, 520, 1024, 1040, 2560, 4096, 4104])
        K = leaf * T
        print("case", it, M, N, K, leaf, flush=True)
        X = O.gaussian_bf16((M, K), 1.0, it).to(dev)
        Wt = O.gaussian_bf16((N, K), 0.02, 1000 + it).to(dev).t()
        full = matmul_tp_persistent(X, Wt, leaf_k=leaf)
        flb = O.tree_params(K, leaf)[1]
        for p in (2, 4, 8):
            # a split is legal when every shard keeps the odd part of the leaf count (or is a single leaf of a pair)
            if T % p == 0 and (O.tree_params(K // p, leaf)[1] == flb or (flb == 2 and T // p == 1)):
                assert_bitwise(sim_tp(X, Wt, p, leaf), full, f"case {it} TP={p}")
        m2 = rng.randint(1, M)
        assert_bitwise(matmul_tp_persistent(X[:m2], Wt, leaf_k=leaf), full[:m2], f"case {it} prefix {m2}")
        i = rng.randrange(M)
        assert_bitwise(matmul_tp_persistent(X[i:i + 1], Wt, leaf_k=leaf), full[i:i + 1], f"case {it} row {i}")


@pytest.mark.parametrize("M,K,N,leaf", [(2048, 12288, 4096, 256), (512, 25600, 5120, 128), (128, 12288, 4096, 256), (1, 12288, 4096, 256)])
def test_repeated_calls_return_the_same_bits(dev, M, K, N, leaf):
    """Run-to-run determinism under load: 25 back-to-back calls (with other work interleaved on the stream) return
    the bits of the first one.  Guards the asynchronous parts of the kernels: direct-to-LDS loads, parked tree levels
    and their read-back, K-cut partials."""
    print("case", M, K, N, leaf, flush=True)
    X = O.gaussian_bf16((M, K), 1.0, 3).to(dev)
    Wt = O.gaussian_bf16((N, K), 0.02, 4).to(dev).t()
    first = matmul_tp_persistent(X, Wt, leaf_k=leaf)
    noise = torch.empty(64 << 20, device=dev, dtype=torch.uint8)
    for i in range(25):
        noise.fill_(i)                     # evicts caches and reuses freed workspaces between the calls
        again = matmul_tp_persistent(X, Wt, leaf_k=leaf)
        assert torch.equal(bits(again), bits(first)), f"call {i} differs"


def test_reference_smoke_script_shape(dev):
    # simple_matmul.py: M,K,N = 1024,6144,2048, both operands ~ N(0,1), row-major B, TP=4, batch halves
    M, K, N = 1024, 6144, 2048
    A = O.gaussian_bf16((M, K), 1.0, 0).to(dev)
    B = O.gaussian_bf16((K, N), 1.0, 1).to(dev)
    C = matmul_tp_persistent(A, B)
    assert_bitwise(matmul_tp_persistent(A[:M // 2], B), C[:M // 2], "batch halves")
    assert_bitwise(sim_tp(A, B, 4, 256), C, "TP=4")
    want = O.matmul_tree(A[:64].cpu(), B.cpu())
    assert_close_to_oracle(C[:64], want, "vs oracle")


def test_tree_combine_matches_oracle_bitwise(dev):
    for numel_shape in [(2048, 4096), (7, 33), (1, 5)]:
        parts = [O.gaussian_bf16(numel_shape, 1.0, s) for s in range(64)]
        for n in (1, 2, 4, 8, 16, 32, 64):
            got = tree_combine([p.to(dev) for p in parts[:n]])
            assert_bitwise(got, O.tree_combine(parts[:n]), f"{numel_shape} n={n}")
    # unaligned views take the scalar path: same bits
    big = O.gaussian_bf16((4, 1001), 1.0, 9)
    views = [big[i, 1:] for i in range(4)]
    assert_bitwise(tree_combine([v.to(dev)[:] for v in views]), O.tree_combine(views), "unaligned")
    flat = big.to(dev).reshape(-1)
    shifted = [flat[1 + i * 1001: 1 + i * 1001 + 999] for i in range(4)]
    assert_bitwise(tree_combine(shifted), O.tree_combine([s.cpu() for s in shifted]), "shifted views")


# ---------------------------------------------------------------------------------------------
# float16: the other 16-bit branch of the reference's dtype-keyed configuration
# (src/tbik/tree_based_matmul.py:206-222): same tree, leaves and nodes rounded to fp16
# ---------------------------------------------------------------------------------------------
def f16_ulp_distance(a, b):
    def ordered(t):
        i = t.contiguous().view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return (ordered(a) - ordered(b)).abs()


def test_fp16_rational_known_answers(dev):
    z = np.load(GOLDEN)
    for n in sorted({k[:-2] for k in z.files if k.endswith("_A")}):
        A = torch.from_numpy(z[n + "_A"].astype(np.float32)).to(torch.float16).to(dev)
        B = torch.from_numpy(z[n + "_B"].astype(np.float32)).to(torch.float16).to(dev)
        C = torch.from_numpy(z[n + "_C16"].view(np.int16).copy()).view(torch.float16)
        leaf = int(z[n + "_leaf"])
        print("fp16 case", n, tuple(A.shape), tuple(B.shape), leaf, flush=True)
        got = matmul_tp_persistent(A, B, leaf_k=leaf)
        assert got.dtype == torch.float16
        assert_bitwise(got, C, n)
        assert_bitwise(matmul_tp_persistent(A, B.t().contiguous().t(), leaf_k=leaf), C, n + " (weight.t())")


@pytest.mark.parametrize("M,N,K,leaf", [(1, 64, 512, 256), (17, 200, 1536, 256), (70, 136, 2048, 256), (300, 520, 3072, 256),
                                        (33, 72, 3200, 128)])
def test_fp16_integer_inputs_match_oracle_bitwise(dev, M, N, K, leaf):
    A = O.integer_bf16((M, K), -9, 9, 3).to(torch.float16)
    W = O.integer_bf16((N, K), -7, 7, 4).to(torch.float16)
    bias = O.integer_bf16((N,), -50, 50, 5).to(torch.float16)
    print("fp16 ints", M, N, K, leaf, flush=True)
    want = O.matmul_tree(A, W.t(), bias, leaf=leaf)
    assert_bitwise(matmul_tp_persistent(A.to(dev), W.to(dev).t(), bias.to(dev), leaf_k=leaf), want, "vs oracle")


def test_fp16_gaussian_tolerance_and_invariance(dev):
    M, K, N = 2048, 4096, 4096
    X = O.gaussian_bf16((M, K), 1.0, 0).to(torch.float16).to(dev)
    W = O.gaussian_bf16((N, K), 0.02, 1).to(torch.float16).to(dev)
    full = matmul_tp_persistent(X, W.t())
    want = O.matmul_tree(X[:64].cpu(), W.cpu().t())
    ulp = f16_ulp_distance(full[:64].cpu(), want)
    diff = (full[:64].cpu().float() - want.float()).abs()
    scale = want.float().abs().max().item()
    bad = (ulp > 1) & (diff > 2.0 ** -11 * scale)   # <= 1 fp16 ulp, or 2^-11 of the output scale
    assert not bad.any(), f"{int(bad.sum())} elements off, max ulp {int(ulp.max())}"
    for p in (2, 4, 8):
        assert_bitwise(sim_tp(X, W.t(), p, 256), full, f"fp16 TP={p}")
    for m in (1, 16, 64, 300):
        assert_bitwise(matmul_tp_persistent(X[:m], W.t()), full[:m], f"fp16 rows {m}")
    parts = [O.gaussian_bf16((33, 257), 1.0, s).to(torch.float16) for s in range(4)]
    assert_bitwise(tree_combine([q.to(dev) for q in parts]), O.tree_combine(parts), "fp16 tree_combine")


# ---------------------------------------------------------------------------------------------
# float32 (leaves of 128, src/tbik/tree_based_matmul.py:223-231)
# ---------------------------------------------------------------------------------------------
def test_fp32_rational_known_answers_and_invariance(dev):
    z = np.load(GOLDEN)
    for n in sorted({k[:-4] for k in z.files if k.endswith("_A32")}):
        A = torch.from_numpy(z[n + "_A32"].astype(np.float32)).to(dev)
        B = torch.from_numpy(z[n + "_B32"].astype(np.float32)).to(dev)
        C = torch.from_numpy(z[n + "_C32"])
        print("fp32 case", n, tuple(A.shape), tuple(B.shape), flush=True)
        got = matmul_tp_persistent(A, B)   # leaf 128 is the float32 default
        assert got.dtype == torch.float32
        assert torch.equal(got.cpu().view(torch.int32), C.view(torch.int32)), n
    M, K, N = 300, 2048, 520
    g = torch.Generator().manual_seed(3)
    X = torch.randn((M, K), generator=g).to(dev)
    W = (torch.randn((N, K), generator=g) * 0.02).to(dev)
    bias = torch.randn((N,), generator=g).to(dev)
    full = matmul_tp_persistent(X, W.t(), bias)
    want = O.matmul_tree(X.cpu(), W.cpu().t(), bias.cpu(), leaf=128)
    assert torch.allclose(full.cpu(), want, rtol=2e-5, atol=2e-5 * want.abs().max().item())
    nb = matmul_tp_persistent(X, W.t())
    for p in (2, 4, 8):
        ks = K // p
        parts = [matmul_tp_persistent(X[:, r * ks:(r + 1) * ks], W[:, r * ks:(r + 1) * ks].t()) for r in range(p)]
        assert torch.equal(tree_combine(parts), nb), f"fp32 TP={p}"
    for m in (1, 17, 64):
        assert torch.equal(matmul_tp_persistent(X[:m], W.t(), bias), full[:m]), f"fp32 rows {m}"


def test_invariance_check_module_honours_the_flag(dev, monkeypatch):
    """`python -m llm_reproducibility_amd.check_matmul`: with TP_INVARIANT_MATMUL=1 both differences are exactly zero
    on the reference's smoke-test shape (simple_matmul.py:6) and on other shard counts; with the flag off the product
    is the vendor library's and the check still runs."""
    from llm_reproducibility_amd import check_matmul
    monkeypatch.setenv("TP_INVARIANT_MATMUL", "1")
    for shards in (2, 4, 8):
        assert check_matmul.run(1024, 6144, 2048, shards) == ("matmul_tp_persistent", 0.0, 0.0), shards
    assert check_matmul.main(["--m", "256", "--k", "4096", "--n", "512", "--shards", "8"]) == 0
    monkeypatch.setenv("TP_INVARIANT_MATMUL", "0")
    name, batch_diff, shard_diff = check_matmul.run(1024, 6144, 2048, 4)
    assert name == "torch.matmul" and batch_diff >= 0.0 and shard_diff >= 0.0


def test_a_host_written_in_c_gets_the_same_properties_through_the_c_abi():
    """tests/c_host/tbik_c_host.c: gcc, the header and the HIP runtime only.  It checks the product against a
    double-precision one, four K shards + shard tree against the unsharded call, a row alone against the row in its
    batch and the workspace-free entry point against the other, the last three bitwise, and exits with 0 when all hold."""
    import subprocess
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_host")
    exe = os.path.join(here, "tbik_c_host")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", here], check=True, capture_output=True)
    print("case C host", exe, flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.strip().endswith("ok"), r.stdout
    assert "4 K shards + shard tree have the bits of the unsharded call" in r.stdout
    assert "without a workspace has the bits of" in r.stdout
