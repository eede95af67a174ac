"""Pins the CPU oracle of the tree matmul (no GPU).

The closed form used everywhere else (`tree_reduce_leaves`) is checked against
  * a symbolic run of `carry_merge`, the line-by-line emulation of the reference's binary-counter loop,
  * the expression the reference's loop is known to produce for T=6 and T=16,
  * the rational-arithmetic known answers in tests/golden (independent rounding code),
  * the plain-C restatement (independent bf16 arithmetic),
  * the reference's own self-checks: batch-slice invariance and simulated-TP invariance are exactly 0.
"""
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import tbik_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kat_tree_matmul.npz")


class Sym:
    """A 'tensor' that records the expression built from clone() and +."""

    def __init__(self, s):
        self.s = s

    def clone(self):
        return Sym(self.s)

    def __add__(self, other):
        return Sym(f"({self.s}+{other.s})")

    def __iadd__(self, other):
        self.s = f"({self.s}+{other.s})"
        return self


def sym_leaves(T):
    return [Sym(f"t{j}") for j in range(T)]


# tree parameters for the shard extents of the benchmark shapes at TP = 1/2/4/8 (leaf 256)
@pytest.mark.parametrize("K,expect", [
    (4096, (16, 2, 4)), (2048, (8, 2, 3)), (1024, (4, 2, 2)), (512, (2, 2, 1)),
    (12288, (48, 3, 5)), (6144, (24, 3, 4)), (3072, (12, 3, 3)), (1536, (6, 3, 2)),
    (8192, (32, 2, 5)), (25600, (100, 25, 3)), (12800, (50, 25, 2)), (6400, (25, 25, 1)),
    (256, (1, 1, 1)), (768, (3, 3, 1)),
])
def test_tree_params(K, expect):
    assert O.tree_params(K) == expect
    assert c_oracle.tree_params(K, 256) == expect
    T, flb, lev = expect
    assert T == flb * 2 ** (lev - 1)


def test_tree_params_rejects_partial_leaf():
    with pytest.raises(AssertionError):
        O.tree_params(3200)          # Qwen3-32B down_proj at TP=8 with leaf 256
    assert O.tree_params(3200, 128) == (25, 25, 1)
    with pytest.raises(ValueError):
        c_oracle.tree_params(3200, 256)


def test_carry_loop_expression_T6_T16():
    # T=6 (FLB=3, two groups): ((t0+t1)+t2)+((t3+t4)+t5)
    assert O.carry_merge(sym_leaves(6), 3, 2).s == "(((t0+t1)+t2)+((t3+t4)+t5))"
    # T=16 (FLB=2): a perfect binary tree of adjacent pairs
    e = O.carry_merge(sym_leaves(16), 2, 4).s
    pairs = [f"(t{2*i}+t{2*i+1})" for i in range(8)]
    quads = [f"({pairs[2*i]}+{pairs[2*i+1]})" for i in range(4)]
    octs = [f"({quads[0]}+{quads[1]})", f"({quads[2]}+{quads[3]})"]
    assert e == f"({octs[0]}+{octs[1]})"


@pytest.mark.parametrize("T", [1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16, 24, 25, 48, 50, 96, 100, 200, 256])
def test_closed_form_equals_carry_loop_symbolically(T):
    flb, lev = T, 1
    while flb > 2 and flb % 2 == 0:
        flb //= 2
        lev += 1
    assert O.tree_reduce_leaves(sym_leaves(T), flb).s == O.carry_merge(sym_leaves(T), flb, lev).s


def test_shard_tree_composes_with_leaf_tree_symbolically():
    # K=12288 at TP=4: each shard has T=12 (FLB=3, 4 groups); the shard tree on top must rebuild the TP=1 tree
    full = O.tree_reduce_leaves(sym_leaves(48), 3).s
    leaves = sym_leaves(48)
    for p in (2, 4, 8):
        per = 48 // p
        parts = [O.tree_reduce_leaves(leaves[r * per:(r + 1) * per], 3) for r in range(p)]
        assert O.tree_combine(parts).s == full, p


def _load_kat():
    z = np.load(GOLDEN)
    names = sorted({k[:-2] for k in z.files if k.endswith("_A")})
    for n in names:
        A = torch.from_numpy(z[n + "_A"].astype(np.float32)).to(torch.bfloat16)
        B = torch.from_numpy(z[n + "_B"].astype(np.float32)).to(torch.bfloat16)
        C = torch.from_numpy(z[n + "_C"].view(np.int16).copy()).view(torch.bfloat16)
        yield n, A, B, C, int(z[n + "_leaf"])


@pytest.mark.parametrize("case", list(_load_kat()), ids=lambda c: c[0])
def test_oracles_reproduce_rational_known_answers(case):
    _, A, B, C, leaf = case
    assert torch.equal(O.matmul_tree(A, B, leaf=leaf).view(torch.int16), C.view(torch.int16))
    assert torch.equal(c_oracle.matmul_tree(A, B, leaf=leaf).view(torch.int16), C.view(torch.int16))


def _load_kat_f16():
    z = np.load(GOLDEN)
    for n in sorted({k[:-2] for k in z.files if k.endswith("_A")}):
        A = torch.from_numpy(z[n + "_A"].astype(np.float32)).to(torch.float16)
        B = torch.from_numpy(z[n + "_B"].astype(np.float32)).to(torch.float16)
        C = torch.from_numpy(z[n + "_C16"].view(np.int16).copy()).view(torch.float16)
        yield n, A, B, C, int(z[n + "_leaf"])


@pytest.mark.parametrize("case", list(_load_kat_f16()), ids=lambda c: c[0])
def test_oracle_reproduces_rational_known_answers_in_fp16(case):
    # the float16 branch of the reference's dtype-keyed configuration (src/tbik/tree_based_matmul.py:206-222):
    # same tree, leaves and nodes rounded to 11 significant bits
    _, A, B, C, leaf = case
    assert torch.equal(O.matmul_tree(A, B, leaf=leaf).view(torch.int16), C.view(torch.int16))


def _load_kat_f32():
    z = np.load(GOLDEN)
    for n in sorted({k[:-4] for k in z.files if k.endswith("_A32")}):
        yield (n, torch.from_numpy(z[n + "_A32"].astype(np.float32)), torch.from_numpy(z[n + "_B32"].astype(np.float32)),
               torch.from_numpy(z[n + "_C32"]))


@pytest.mark.parametrize("case", list(_load_kat_f32()), ids=lambda c: c[0])
def test_oracle_reproduces_rational_known_answers_in_fp32(case):
    # float32 branch (leaves of 128, src/tbik/tree_based_matmul.py:223-231): one exact product per leaf, sums
    # beyond 2^24, so only the tree order and fp32 rounding decide the bits
    _, A, B, C = case
    assert torch.equal(O.matmul_tree(A, B, leaf=128).view(torch.int32), C.view(torch.int32))


def test_known_answers_discriminate_other_orders():
    # a sequential (left-to-right over all leaves) order or an fp32 tree must NOT reproduce the fixtures
    differs_seq = differs_f32 = 0
    for _, A, B, C, leaf in _load_kat():
        leaves = O.leaf_partials(A, B, leaf)
        seq = leaves[0].clone()
        for t in leaves[1:]:
            seq = seq + t
        f32 = (A.float() @ B.float()).to(torch.bfloat16)
        differs_seq += int(not torch.equal(seq, C))
        differs_f32 += int(not torch.equal(f32, C))
    assert differs_seq >= 3 and differs_f32 >= 5


@pytest.mark.parametrize("seed", [0, 1])
def test_c_and_torch_oracles_agree_on_integer_inputs(seed):
    A = O.integer_bf16((6, 3072), -8, 8, seed)
    B = O.integer_bf16((3072, 24), -6, 6, seed + 100)
    bias = O.integer_bf16((24,), -50, 50, seed + 200)
    for leaf in (256, 128):
        assert torch.equal(O.matmul_tree(A, B, bias, leaf=leaf), c_oracle.matmul_tree(A, B, bias, leaf=leaf))


def test_tree_combine_oracles_agree_and_reject_non_power_of_two():
    parts = [O.gaussian_bf16((33, 17), 1.0, s) for s in range(8)]
    for n in (1, 2, 4, 8):
        assert torch.equal(O.tree_combine(parts[:n]), c_oracle.tree_combine(parts[:n]))
    with pytest.raises(ValueError):
        O.tree_combine(parts[:3])
    with pytest.raises(ValueError):
        c_oracle.tree_combine(parts[:6])
    # ((p0+p1)+(p2+p3)) by hand
    want = (parts[0] + parts[1]) + (parts[2] + parts[3])
    assert torch.equal(O.tree_combine(parts[:4]), want)


def test_reference_self_checks_hold_on_config1():
    # A[256,4096] ~ N(0,1), W[4096,4096] ~ N(0,0.02), seed 0; TP 1/2/4/8 must be bitwise identical
    A = O.gaussian_bf16((256, 4096), 1.0, 0)
    W = O.gaussian_bf16((4096, 4096), 0.02, 1)
    full = O.matmul_tree(A, W)
    for p in (2, 4, 8):
        assert torch.equal(O.simulated_tp_matmul(A, W, p), full), p
    # batch-slice invariance (simple_matmul.py:16-20)
    assert torch.equal(O.matmul_tree(A[:128], W), full[:128])
    # and the tree result stays close to the fp32 product (K=leaf special case is exactly one rounding)
    ref = A.float() @ W.float()
    assert (full.float() - ref).abs().max() <= 2 ** -6 * ref.abs().max()
    one_leaf = O.matmul_tree(A[:, :256], W[:256])
    assert torch.equal(one_leaf, (A[:, :256].float() @ W[:256].float()).to(torch.bfloat16))


def test_zero_leaves_at_aligned_positions_do_not_change_the_result():
    # appending a zero subtree of equal size: x + 0 == x at every node
    A = O.gaussian_bf16((4, 1024), 1.0, 3)
    W = O.gaussian_bf16((1024, 8), 0.05, 4)
    Az = torch.cat([A, torch.zeros_like(A)], dim=1)
    Wz = torch.cat([W, torch.zeros_like(W)], dim=0)
    assert torch.equal(O.matmul_tree(Az, Wz), O.matmul_tree(A, W))


def test_row_permutation_commutes():
    A = O.gaussian_bf16((16, 768), 1.0, 5)
    W = O.gaussian_bf16((768, 8), 0.05, 6)
    perm = torch.randperm(16, generator=torch.Generator().manual_seed(0))
    assert torch.equal(O.matmul_tree(A[perm], W), O.matmul_tree(A, W)[perm])
