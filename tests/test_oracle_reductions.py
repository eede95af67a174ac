"""Pins the CPU oracles of the batch-invariant reductions against library routines and closed forms (no GPU)."""
import math
from fractions import Fraction

import pytest
import torch

from oracle import tbik_oracle as O


def test_log_softmax_matches_float64_library_and_closed_forms():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((7, 151936), generator=g) * 3.0
    want = torch.log_softmax(x.double(), dim=-1)
    got = O.log_softmax_lastdim(x)
    assert (got.double() - want).abs().max() < 2e-5
    # constant row: -log(V) everywhere
    c = torch.full((2, 1000), 4.25)
    assert torch.allclose(O.log_softmax_lastdim(c), torch.full((2, 1000), -math.log(1000.0)), atol=1e-6)
    # one dominant entry: ~0 there, ~(x - big) elsewhere
    d = torch.zeros((1, 64))
    d[0, 5] = 100.0
    r = O.log_softmax_lastdim(d)
    assert abs(r[0, 5].item()) < 1e-6 and abs(r[0, 0].item() + 100.0) < 1e-4
    # (the CPU library reduction is itself not batch invariant -- its blocking depends on the shape --
    # so rows computed alone agree with rows computed in a batch only to rounding)
    assert (O.log_softmax_lastdim(x[2:3]) - got[2:3]).abs().max() < 1e-5


def test_mean_matches_integers_and_float64():
    x = torch.arange(0, 4096, dtype=torch.float32).repeat(3, 1)
    assert torch.equal(O.mean_lastdim(x), torch.full((3,), 2047.5))
    g = torch.Generator().manual_seed(1)
    y = torch.randn((5, 4096), generator=g)
    assert (O.mean_lastdim(y).double() - y.double().mean(-1)).abs().max() < 1e-6


def test_rmsnorm_matches_textbook_float64_and_hf_module():
    x = O.gaussian_bf16((9, 4096), 1.0, 2)
    w = (1.0 + 0.1 * torch.randn(4096, generator=torch.Generator().manual_seed(3))).to(torch.bfloat16)
    eps = 1e-6
    got = O.rmsnorm(x, w, eps)
    xd = x.double()
    want = xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + eps)
    want = want.to(torch.bfloat16).double() * w.double()
    assert O.bf16_ulp_distance(got, want.to(torch.bfloat16)).max() <= 1
    # Hugging Face's Qwen3RMSNorm (installed library, same published formula up to where the weight is applied)
    tr = pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    mod = tr.Qwen3RMSNorm(4096, eps=eps)
    with torch.no_grad():
        mod.weight.copy_(w.float())
    hf = mod(x.float())
    assert (got.float() - hf).abs().max() <= 2 ** -7 * hf.abs().max()
    # +-1 row, unit weight: x * rsqrt(1 + eps)
    s = torch.ones((1, 4096), dtype=torch.bfloat16)
    s[0, ::2] = -1
    r = O.rmsnorm(s, torch.ones(4096, dtype=torch.bfloat16), eps)
    assert torch.equal(r, s)


def test_rmsnorm_residual_semantics():
    x = O.gaussian_bf16((4, 512), 1.0, 4)
    res = O.gaussian_bf16((4, 512), 1.0, 5)
    w = torch.ones(512, dtype=torch.bfloat16)
    y, new_res = O.rmsnorm(x, w, 1e-6, residual=res)
    assert torch.equal(new_res, (x.float() + res.float()).to(torch.bfloat16))
    s = x.float() + res.float()          # the normalisation sees the UNROUNDED fp32 sum
    want = (s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    assert torch.equal(y, want)


def _rne_bf16(x: Fraction) -> float:
    """Round an exact rational to the nearest bf16 (8 significant bits), ties to even -- integer arithmetic only."""
    if x == 0:
        return 0.0
    sign = -1 if x < 0 else 1
    x = abs(x)
    e = 0
    while x >= 256:          # scale into [128, 256): 8 significant bits are then the integer part
        x /= 2
        e += 1
    while x < 128:
        x *= 2
        e -= 1
    n = x.numerator // x.denominator
    rem = x - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return float(sign * Fraction(n) * Fraction(2) ** e)


def rounding_point_case():
    """A row whose normalisation is exact rational arithmetic: the pattern (1,2,3,4,5,6,7,2,0 x 8) has mean(x^2) = 9,
    so with eps = 0 the factor is exactly 1/3; repeated 128 times, with column block b weighted by the bf16 value
    1 + b/128 (every bf16 in [1, 2)).  Returns x [1, 2048], w [2048] and, from exact fractions with an independent
    round-to-nearest-even, the result of (a) rounding x/3 to bf16 and then multiplying by w in bf16 -- the documented
    order, vLLM's `x.to(orig_dtype) * weight` -- and (b) multiplying in full precision and rounding once."""
    pat = [1, 2, 3, 4, 5, 6, 7, 2] + [0] * 8
    x = torch.tensor([pat * 128], dtype=torch.float32).to(torch.bfloat16)
    w = torch.tensor([1.0 + b / 128.0 for b in range(128) for _ in range(16)], dtype=torch.float32).to(torch.bfloat16)
    two, one = [], []
    for b in range(128):
        wb = Fraction(128 + b, 128)
        for v in pat:
            two.append(_rne_bf16(Fraction(_rne_bf16(Fraction(v, 3))) * wb))
            one.append(_rne_bf16(Fraction(v, 3) * wb))
    as_bf16 = lambda vals: torch.tensor([vals], dtype=torch.float64).to(torch.bfloat16)  # noqa: E731  (exact: already bf16 values)
    return x, w, as_bf16(two), as_bf16(one)


def test_rmsnorm_rounds_to_the_input_type_before_the_weight_multiply():
    x, w, two_roundings, one_rounding = rounding_point_case()
    differ = (two_roundings != one_rounding).sum().item()
    assert differ > 100, differ                       # the case separates the two orders on many elements
    got = O.rmsnorm(x, w, 0.0)
    assert torch.equal(got, two_roundings)
    assert not torch.equal(got, one_rounding)
    # the same with a residual: x = r = half the pattern, so the fp32 sum is the pattern again, and a NON-unit weight
    half = (x.float() / 2).to(torch.bfloat16)
    y, new_res = O.rmsnorm(half, w, 0.0, residual=half)
    assert torch.equal(new_res, x) and torch.equal(y, two_roundings)


def test_single_accumulator_matmul_against_exact_rational_arithmetic():
    # integer operands: every product and every partial sum is an integer below 2^24, so an fp32 accumulator is exact
    # in ANY order and the result is one rounding of the exact sum (+ bias); sums reach the thousands, so an
    # accumulator with fewer bits (bf16: 8, fp16: 11) cannot reproduce them
    a = O.integer_bf16((6, 320), -9, 9, 11)
    b = O.integer_bf16((320, 5), -7, 7, 12)
    bias = O.integer_bf16((5,), -300, 300, 13)          # multiples of 2 above 256 are bf16 values; make them so
    bias = (bias.float() / 4).round().mul(4).to(torch.bfloat16)
    got = O.matmul_single_acc(a, b, bias)
    ai, bi, ci = a.double().long().tolist(), b.double().long().tolist(), bias.double().long().tolist()
    big = 0
    for m in range(6):
        for n in range(5):
            exact = sum(ai[m][k] * bi[k][n] for k in range(320)) + ci[n]
            big = max(big, abs(exact))
            assert got[m, n].item() == _rne_bf16(Fraction(exact)), (m, n, exact)
    assert big > 512                                     # the rounding is exercised, not only exact values
    nb = O.matmul_single_acc(a, b)
    for m in range(6):
        for n in range(5):
            assert nb[m, n].item() == _rne_bf16(Fraction(sum(ai[m][k] * bi[k][n] for k in range(320))))


def test_single_accumulator_matmul_adds_the_bias_before_the_one_rounding():
    # sum = 257 (needs rounding: bf16 has 256 and 258), bias = 1.  Bias BEFORE the rounding (the reference adds it to
    # the fp32 accumulator, src/bio/batch_invariant_ops.py:115-118): 258, exact.  Bias AFTER: bf16(257) = 256 (tie to
    # even), 256 + 1 = 257 -> 256.  The two differ, the oracle must give the first.
    a = torch.zeros((1, 264), dtype=torch.bfloat16)
    a[0, :257] = 1
    b = torch.ones((264, 1), dtype=torch.bfloat16)
    bias = torch.ones((1,), dtype=torch.bfloat16)
    assert O.matmul_single_acc(a, b, bias).item() == 258.0
    after = (O.matmul_single_acc(a, b) + bias).item()
    assert after == 256.0                                # what a bias applied to the rounded output would give


def test_single_accumulator_matmul_rounds_once_not_through_fp16():
    # 1 + 2^-8 + 2^-12: straight to bf16 it lies above the midpoint of 1 and 1 + 2^-7 -> rounds up.  Through fp16 first
    # (the reference's detour, src/bio/batch_invariant_ops.py:119-123) the 2^-12 is lost, the value becomes the
    # midpoint itself and the tie goes to 1.0; and anything above 65504 becomes inf.  The documented choice here is the
    # single rounding.
    a = torch.tensor([[1.0, 2.0 ** -8, 2.0 ** -12, 0, 0, 0, 0, 0]], dtype=torch.bfloat16)
    b = torch.ones((8, 1), dtype=torch.bfloat16)
    got = O.matmul_single_acc(a, b).item()
    assert got == 1.0 + 2.0 ** -7
    detour = (a.float() @ b.float()).half().to(torch.bfloat16).item()
    assert detour == 1.0 and detour != got
    big = torch.full((1, 8), 128.0, dtype=torch.bfloat16)
    bb = torch.full((8, 1), 128.0, dtype=torch.bfloat16)
    assert O.matmul_single_acc(big, bb).item() == 131072.0 and math.isinf((big.float() @ bb.float()).half().item())
    # fp16 operands: the same single rounding to fp16
    ah, bh = O.gaussian_bf16((5, 64), 1.0, 20).half(), O.gaussian_bf16((64, 3), 1.0, 21).half()
    want = (ah.double() @ bh.double())
    assert ((O.matmul_single_acc(ah, bh).double() - want).abs() <= want.abs() * 2.0 ** -11 + 1e-6).all()


def test_silu_mul_matches_library_float64_and_closed_forms():
    g = torch.Generator().manual_seed(5)
    gu = (torch.randn((33, 512), generator=g) * 3).to(torch.bfloat16)
    got = O.silu_mul(gu)
    assert got.shape == (33, 256) and got.dtype == torch.bfloat16
    # library routine on the same bf16 tensors (two roundings: silu, then the product)
    lib = torch.nn.functional.silu(gu[:, :256]) * gu[:, 256:]
    assert O.bf16_ulp_distance(got, lib).max().item() <= 1
    # float64 evaluation with the two roundings applied explicitly
    g64 = gu[:, :256].double()
    s = (g64 / (1 + torch.exp(-g64))).to(torch.bfloat16)
    want = (s.double() * gu[:, 256:].double()).to(torch.bfloat16)
    assert O.bf16_ulp_distance(got, want).max().item() <= 1
    # closed forms: silu(0) = 0; silu(x) = x once exp(-x) underflows against 1; silu(-large) = -0 * ... = 0
    gu = torch.tensor([[0.0, 40.0, -100.0, 2.0, 2.0, 2.0]], dtype=torch.bfloat16)
    assert O.silu_mul(gu).tolist() == [[0.0, 80.0, -0.0]]
