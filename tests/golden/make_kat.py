"""Writes the integer known-answer fixtures for the tree matmul (tests/golden/kat_tree_matmul.npz).

Inputs are small integers, so every leaf sum is an integer that fp32 holds exactly in ANY
accumulation order; the expected output is then a function of the tree order and of round-to-
nearest-even alone, and any implementation of the contract must reproduce it bit for bit.
Expected values come from the rational-arithmetic brute force below (exact leaf sums as Python
integers, explicit bf16 rounding), which shares no code with oracle/.

    python tests/golden/make_kat.py
"""
import os
import sys
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def rn(x: Fraction, sig_bits: int) -> Fraction:
    """Round a rational to `sig_bits` significant bits (8: bf16, 11: fp16), ties to even; no overflow or
    subnormal handling (the callers check the range)."""
    if x == 0:
        return Fraction(0)
    s = -1 if x < 0 else 1
    a = abs(x)
    e = 0
    while a >= 2 ** (e + 1):
        e += 1
    while a < 2 ** e:
        e -= 1
    ulp = Fraction(2) ** (e - (sig_bits - 1))
    q = a / ulp
    fl = q.numerator // q.denominator
    rem = q - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return s * fl * ulp


def tree_params(T):
    flb, lev = T, 1
    while flb > 2 and flb % 2 == 0:
        flb //= 2
        lev += 1
    return flb, lev


def brute_force(A, B, leaf, sig_bits):
    M, K = A.shape
    N = B.shape[1]
    T = K // leaf
    flb, _ = tree_params(T)
    out = np.zeros((M, N), dtype=np.float64)
    for m in range(M):
        for n in range(N):
            leaves = [rn(Fraction(int(np.dot(A[m, j * leaf:(j + 1) * leaf], B[j * leaf:(j + 1) * leaf, n]))), sig_bits)
                      for j in range(T)]
            groups = []
            for g in range(0, T, flb):
                s = leaves[g]
                for j in range(1, flb):
                    s = rn(s + leaves[g + j], sig_bits)
                groups.append(s)
            while len(groups) > 1:
                groups = [rn(groups[i] + groups[i + 1], sig_bits) for i in range(0, len(groups), 2)]
            out[m, n] = float(groups[0])
    return out


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    f = x.astype(np.float32)
    assert np.array_equal(f.astype(np.float64), x), "value not exact in fp32"
    u = f.view(np.uint32)
    assert np.all((u & 0xFFFF) == 0), "value not exact in bf16"
    return (u >> 16).astype(np.uint16)


def to_f16_bits(x: np.ndarray) -> np.ndarray:
    assert np.abs(x).max() < 65504, "fp16 overflow: outside what the brute force models"
    h = x.astype(np.float16)
    assert np.array_equal(h.astype(np.float64), x), "value not exact in fp16"
    return h.view(np.uint16)


CASES = [  # name, M, N, K, leaf, amax, bmax, seed
    ("t1_flb1", 5, 8, 256, 256, 9, 7, 1),
    ("t2_flb2", 4, 8, 512, 256, 9, 7, 2),
    ("t3_flb3", 4, 8, 768, 256, 9, 7, 3),
    ("t6_flb3_l2", 3, 8, 1536, 256, 9, 7, 4),
    ("t8_flb2_l3", 3, 8, 2048, 256, 9, 7, 5),
    ("t5_flb5", 3, 8, 1280, 256, 9, 7, 6),
    ("t12_leaf128", 3, 8, 1536, 128, 9, 7, 7),
    ("t25_leaf128", 2, 8, 3200, 128, 9, 7, 8),
    ("t48_flb3_l5", 2, 4, 12288, 256, 9, 7, 9),
]


# float32 (leaves of 128, 24 significant bits): ONE non-zero product per leaf, so every leaf is exact whatever the
# order inside it, and products near 2^24 so that the nodes above do round: the result pins the tree order.
CASES_F32 = [  # name, M, N, K, seed
    ("f32_t6_flb3", 3, 4, 768, 11),
    ("f32_t16_flb2", 3, 4, 2048, 12),
    ("f32_t25_flb25", 2, 4, 3200, 13),
    ("f32_t48_flb3", 2, 4, 6144, 14),
]


def main():
    out = {}
    for name, M, N, K, seed in CASES_F32:
        rng = np.random.default_rng(seed)
        A = np.zeros((M, K), dtype=np.int64)
        B = np.zeros((K, N), dtype=np.int64)
        for j in range(K // 128):
            pos = j * 128 + int(rng.integers(0, 128))
            A[:, pos] = rng.integers(1, 4096, size=M) * rng.choice([-1, 1], size=M)
            B[pos, :] = rng.integers(1, 4096, size=N) * rng.choice([-1, 1], size=N)
        C = brute_force(A, B, 128, 24)
        seq = np.zeros_like(C)
        for m in range(M):
            for n in range(N):
                acc = Fraction(0)
                for j in range(K // 128):
                    acc = rn(acc + int(np.dot(A[m, j * 128:(j + 1) * 128], B[j * 128:(j + 1) * 128, n])), 24)
                seq[m, n] = float(acc)
        assert np.array_equal(C.astype(np.float32).astype(np.float64), C)
        out[name + "_A32"] = A.astype(np.int16)
        out[name + "_B32"] = B.astype(np.int16)
        out[name + "_C32"] = C.astype(np.float32)
        print(name, "max |C| =", np.abs(C).max(), "nodes round:", bool(np.abs(C).max() > 2 ** 24),
              "differs from a sequential fp32 sum:", bool((C != seq).any()))
    for name, M, N, K, leaf, amax, bmax, seed in CASES:
        rng = np.random.default_rng(seed)
        A = rng.integers(-amax, amax + 1, size=(M, K)).astype(np.int64)
        B = rng.integers(-bmax, bmax + 1, size=(K, N)).astype(np.int64)
        C = brute_force(A, B, leaf, 8)
        C16 = brute_force(A, B, leaf, 11)
        out[name + "_A"] = A.astype(np.int8)
        out[name + "_B"] = B.astype(np.int8)
        out[name + "_C"] = to_bf16_bits(C)
        out[name + "_C16"] = to_f16_bits(C16)   # the same product with fp16 leaves and nodes
        out[name + "_leaf"] = np.array(leaf, dtype=np.int32)
        print(name, "max |C| =", np.abs(C).max(), "rounded nodes matter:", bool(np.abs(C).max() > 256),
              "| fp16:", bool(np.abs(C16).max() > 2048), "differs from bf16:", bool((C != C16).any()))
    np.savez_compressed(os.path.join(HERE, "kat_tree_matmul.npz"), **out)


if __name__ == "__main__":
    sys.exit(main())
