"""CPU oracle for the tree-ordered (TP-invariant) matmul and the batch-invariant reductions.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module: it is the
checker for the HIP kernels (tests, the smoke check and the CPU-baseline leg of the benchmark),
never the thing that is measured or shipped.

Every function restates, on the CPU with plain PyTorch, the arithmetic of one piece of the
reference and cites the lines it follows (paths relative to the reference checkout):

* tree parameters ............ src/tbik/tree_based_matmul.py:240-249
* leaf value ................. src/tbik/tree_based_matmul.py:121-136   (fp32 dot over one K chunk -> bf16)
* carry / merge loop ......... src/tbik/tree_based_matmul.py:140-174   (literal emulation: `carry_merge`)
* closed form of that loop ... `tree_reduce_leaves` (level 0 left-to-right over FLB leaves, then adjacent pairs)
* shard combine .............. src/tbik/tree_based_all_reduce.py:32-35, simple_matmul.py:35-38,
                               mini_allreduce/tbik_kernel/csrc/allreduce/custom_all_reduce.cuh:203-234
* simulated TP ............... simple_matmul.py:23-43
* batch-invariant mm ......... src/bio/batch_invariant_ops.py:98-123   (one fp32 accumulator over all of K)
* log_softmax ................ src/bio/batch_invariant_ops.py:219-260
* mean ....................... src/bio/batch_invariant_ops.py:331-349
* RMSNorm .................... src/patch/patch_batch_invariant.py:9-16 -> vLLM RMSNorm.forward_native
                               (vllm==0.11.0 is not vendored in the reference; the public formula is restated)
* causal attention ........... src/patch/patch_training_inference_align.py:171-487 (what the fixed-order kernel
                               computes: softmax(q k^T * scale, causal) v per head, grouped-query heads)
* rotary embedding ........... src/patch/patch_training_inference_align.py:35-44 (inverse frequencies in fp32 on
                               the CPU) + the rotate-half form of the engine that the reference drives
* greedy token choice ........ simple_inference.py:62-105 (sampling inside the engine; the tie rule -- lowest
                               index -- is this build's, the reference leaves it to the library)

Pin status (what checks each function independently of its own formula; see tests/test_oracle_*.py):

* `tree_params`, `tree_reduce_leaves`, `tree_combine`: pinned.  The closed form is checked against
  `carry_merge` (a line-by-line emulation of the reference's binary-counter loop), against an exact
  rational-arithmetic brute force with an independent round-to-nearest-even, against the plain-C
  restatement in oracle/tbik_oracle.c, and through the reference's own self-consistency checks
  (simple_matmul.py:16-43: batch-slice invariance and simulated-TP invariance must be exactly 0).
* `leaf_partials`: the intra-chunk fp32 accumulation order is hardware defined in the reference
  (Triton `tl.dot`), so it is pinned bit-exactly only where the chunk sum is exactly representable
  (integer-valued inputs), and to 1 bf16 ulp otherwise.  PARITY UNPINNED beyond that.
* `rmsnorm`: PARITY UNPINNED against the reference (the arithmetic lives in vllm==0.11.0, absent);
  pinned to the textbook formula in float64 and to closed-form cases.
* `silu_mul`: PARITY UNPINNED against the reference (vLLM's SiluAndMul is absent); pinned to the
  library routine `torch.nn.functional.silu` (bit-equal on bf16 inputs up to 1 ulp of the device exp),
  to closed forms (silu(0) = 0, silu(x) -> x for large x) and to a float64 evaluation.
* `log_softmax`, `mean_lastdim`: pinned to float64 library routines and closed-form cases; the
  reference's in-block reduction order (Triton `tl.sum`) is backend defined, so tolerance only.
* `matmul_single_acc`: pinned by exact rational arithmetic with an independent round-to-nearest-even on
  integer operands (any accumulation narrower than fp32 fails it), by a case in which a bias added
  before the rounding and one added after it give different bits, and by a case in which the
  reference's detour through fp16 (src/bio/batch_invariant_ops.py:119-123) gives different bits -- the
  single rounding is the documented choice.
* `causal_attention`, `rotate_half_rope`, `qk_norm_rope`, `argmax_lowest_index`: pinned to the library
  routine `torch.nn.functional.scaled_dot_product_attention` in float64, to closed forms (uniform
  scores -> running mean of V, a dominant key -> its value, rotation by pi/2 and by 0, norm
  preservation) and to brute force; the reference's own kernels for them (Triton unified attention,
  vLLM rotary embedding and sampler) are backend defined or absent, so tolerance only: PARITY UNPINNED
  at the bit level.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

LEAF_BF16 = 256  # BLOCK_SIZE_K of the bf16/fp16 configs, src/tbik/tree_based_matmul.py:206-222


# --------------------------------------------------------------------------------------------
# tree shape
# --------------------------------------------------------------------------------------------
def tree_params(K: int, leaf: int = LEAF_BF16) -> Tuple[int, int, int]:
    """(T, FLB, LEVEL_K) for a K extent, following src/tbik/tree_based_matmul.py:242-249.

    T leaves of `leaf` elements; FLB = T with factors of two removed while it is even and > 2;
    LEVEL_K = number of halvings + 1, so T == FLB * 2**(LEVEL_K-1).
    """
    assert K % leaf == 0, "K must be a whole number of leaves"
    T = K // leaf
    flb, level_k = T, 1
    while flb > 2 and flb % 2 == 0:
        flb //= 2
        level_k += 1
    return T, flb, level_k


# --------------------------------------------------------------------------------------------
# leaves
# --------------------------------------------------------------------------------------------
def leaf_partials(A: torch.Tensor, B: torch.Tensor, leaf: int = LEAF_BF16) -> List[torch.Tensor]:
    """One bf16 [M,N] partial per K chunk: fp32 dot over the chunk, rounded once to A's dtype.

    Follows src/tbik/tree_based_matmul.py:121-136 (`acc = tl.dot(a, b).to(ACC_DTYPE)` with
    ACC_DTYPE = A.dtype, :193-194).
    """
    M, K = A.shape
    assert B.shape[0] == K
    out = []
    for k0 in range(0, K, leaf):
        a = A[:, k0:k0 + leaf].float()
        b = B[k0:k0 + leaf, :].float()
        out.append(torch.matmul(a, b).to(A.dtype))
    return out


# --------------------------------------------------------------------------------------------
# merge order: literal emulation and closed form
# --------------------------------------------------------------------------------------------
def carry_merge(leaves: Sequence[torch.Tensor], flb: int, level_k: int) -> torch.Tensor:
    """Line-by-line emulation of the binary-counter loop, src/tbik/tree_based_matmul.py:119-174.

    `count[level]` is the number of partials absorbed at that level; level 0 carries when it has
    absorbed FLB leaves, every other level when it has absorbed 2.  Partials of levels 0..2 live in
    acc1..acc3, deeper ones in S[level-3].  All adds are in the tensors' dtype (bf16).
    """
    manual_acc = 3
    count = [0] * max(level_k, 1)
    acc1 = acc2 = acc3 = None
    S = {}
    acc = None
    for leaf in leaves:
        acc = leaf.clone()
        break_flag = False
        for level in range(level_k):
            if break_flag:
                continue
            count_value_added = count[level] + 1
            table_value = flb if level == 0 else 2
            carry_over = table_value == count_value_added
            if count_value_added > 1:
                if level == 0:
                    acc = acc1 + acc
                elif level == 1:
                    acc = acc2 + acc
                elif level == 2:
                    acc = acc3 + acc
                else:
                    acc = S[level - manual_acc] + acc
            count[level] = 0 if carry_over else count_value_added
            if not carry_over:
                break_flag = True
                if level == 0:
                    acc1 = acc
                elif level == 1:
                    acc2 = acc
                elif level == 2:
                    acc3 = acc
                else:
                    S[level - manual_acc] = acc
    return acc


def tree_combine(parts: Sequence[torch.Tensor]) -> torch.Tensor:
    """Adjacent-pair binary tree over a power-of-two number of partials, adds in the parts' dtype.

    Follows src/tbik/tree_based_all_reduce.py:26-37 (and simple_matmul.py:35-38,
    custom_all_reduce.cuh:203-234): at level l, result[left] += result[left + 2**(l-1)].
    """
    n = len(parts)
    if n & (n - 1) != 0 or n == 0:
        raise ValueError("the number of partials must be a power of two")
    result = [p.clone() for p in parts]
    for level in range(1, n.bit_length()):
        for left in range(0, n, 1 << level):
            right = left + (1 << (level - 1))
            result[left] += result[right]
    return result[0]


def tree_reduce_leaves(leaves: Sequence[torch.Tensor], flb: int) -> torch.Tensor:
    """Closed form of `carry_merge`: left-to-right sums of FLB consecutive leaves, then `tree_combine`."""
    assert len(leaves) % flb == 0
    groups = []
    for g in range(0, len(leaves), flb):
        s = leaves[g].clone()
        for j in range(1, flb):
            s = s + leaves[g + j]
        groups.append(s)
    return tree_combine(groups)


# --------------------------------------------------------------------------------------------
# the operator and the simulated tensor-parallel harness
# --------------------------------------------------------------------------------------------
def matmul_tree(A: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor] = None,
                leaf: int = LEAF_BF16) -> torch.Tensor:
    """CPU restatement of matmul_tp_persistent (src/tbik/tree_based_matmul.py:190-277)."""
    assert A.shape[-1] == B.shape[-2], "Dim doesn't match"
    _, flb, _ = tree_params(A.shape[1], leaf)
    C = tree_reduce_leaves(leaf_partials(A, B, leaf), flb)
    if bias is not None:
        C += bias  # :275-276, added in the output dtype after the tree
    return C


def simulated_tp_matmul(A: torch.Tensor, B: torch.Tensor, num_shards: int,
                        leaf: int = LEAF_BF16) -> torch.Tensor:
    """K split into `num_shards` equal contiguous slices, one tree matmul each, then the shard tree.

    Follows simple_matmul.py:23-38 (with the shard count no longer hard-coded to 4).
    """
    K = A.shape[1]
    assert K % num_shards == 0
    ks = K // num_shards
    parts = [matmul_tree(A[:, i * ks:(i + 1) * ks], B[i * ks:(i + 1) * ks, :], leaf=leaf)
             for i in range(num_shards)]
    return tree_combine(parts)


# --------------------------------------------------------------------------------------------
# batch-invariant ops
# --------------------------------------------------------------------------------------------
def matmul_single_acc(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Batch-invariant mm/addmm: one fp32 accumulator over all of K, bias added in fp32, one rounding.

    Follows src/bio/batch_invariant_ops.py:98-118.  The reference then rounds through fp16 before the
    store converts to the output dtype (:119-123); that detour is deliberately not reproduced, the
    result here is rounded once to the output dtype.
    """
    acc = torch.matmul(a.float(), b.float())
    if bias is not None:
        acc = acc + bias.float()
    return acc.to(a.dtype)


def log_softmax_lastdim(x: torch.Tensor) -> torch.Tensor:
    """x - max - log(sum(exp(x - max))) per row in fp32; src/bio/batch_invariant_ops.py:219-260."""
    xf = x.float()
    m = xf.max(dim=-1, keepdim=True).values
    s = torch.exp(xf - m).sum(dim=-1, keepdim=True)
    return (xf - m - torch.log(s)).to(x.dtype)


def mean_lastdim(x: torch.Tensor, keepdim: bool = False) -> torch.Tensor:
    """fp32 sum over the last dim divided by its length; src/bio/batch_invariant_ops.py:331-349."""
    n = x.shape[-1]
    return (x.float().sum(dim=-1, keepdim=keepdim) / n).to(x.dtype)


def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float,
            residual: Optional[torch.Tensor] = None):
    """RMSNorm as vLLM's RMSNorm.forward_native computes it (reached through
    src/patch/patch_batch_invariant.py:9-16; vllm==0.11.0 itself is not in the reference tree).

    x -> fp32; optional `x += residual` with the sum rounded to the input dtype as the new residual;
    var = mean(x^2) over the last dim; x * rsqrt(var + eps) rounded to the input dtype, THEN
    multiplied by the weight in the input dtype.
    """
    orig = x.dtype
    xf = x.float()
    new_residual = None
    if residual is not None:
        xf = xf + residual.float()
        new_residual = xf.to(orig)
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    y = (xf * torch.rsqrt(var + eps)).to(orig)
    if weight is not None:
        y = y * weight
    return y if residual is None else (y, new_residual)


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """act = silu(gate) * up for gate_up = [gate | up] on the last dimension, the way an unfused
    `F.silu(gate) * up` on bf16 tensors rounds: silu in fp32 rounded to the input dtype, then the product
    rounded again.  This is the producer of down_proj's input (the patched RowParallelLinear forward,
    src/patch/patch_tp_invariant.py:10-48); the activation itself lives in vLLM (not in the reference tree).
    """
    inter = gate_up.shape[-1] // 2
    g, u = gate_up[..., :inter].float(), gate_up[..., inter:]
    s = (g / (1.0 + torch.exp(-g))).to(gate_up.dtype)
    return s * u


# --------------------------------------------------------------------------------------------
# attention, rotary embedding, greedy choice (the callers either side of the row-split GEMM)
# --------------------------------------------------------------------------------------------
def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """Textbook causal grouped-query attention of ONE sequence in float64.

    q [n, Hq, D] are the LAST n positions of the sequence whose keys / values are k, v [L, Hkv, D]
    (n == L: prefill; n == 1: decode; 1 < n < L: chunked prefill).  Query head h reads KV head
    h // (Hq // Hkv).  Returns float64 [n, Hq, D]: softmax over the keys at positions <= the query's,
    then the weighted sum of the values.  This is what _kernel_unified_attention_2d computes per
    (query, head) (src/patch/patch_training_inference_align.py:171-487), without its tiling.
    """
    n, Hq, D = q.shape
    L, Hkv, _ = k.shape
    assert Hq % Hkv == 0 and n <= L
    rep = Hq // Hkv
    qd, kd, vd = q.double(), k.double(), v.double()
    out = torch.empty((n, Hq, D), dtype=torch.float64)
    for h in range(Hq):
        kh, vh = kd[:, h // rep], vd[:, h // rep]              # [L, D]
        s = (qd[:, h] @ kh.t()) * scale                        # [n, L]
        qpos = torch.arange(L - n, L)[:, None]
        s = s.masked_fill(torch.arange(L)[None, :] > qpos, float("-inf"))
        s = s - s.max(dim=-1, keepdim=True).values
        p = torch.exp(s)
        out[:, h] = (p / p.sum(dim=-1, keepdim=True)) @ vh
    return out


def rope_inv_freq(rotary_dim: int, base: float) -> torch.Tensor:
    """fp32 inverse frequencies computed on the CPU, src/patch/patch_training_inference_align.py:36-41."""
    arange = torch.arange(0, rotary_dim, 2, dtype=torch.float)
    return 1.0 / (base ** (arange / rotary_dim))


def rotate_half_rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """Rotate-half rotary embedding: channel pair (i, i + D/2) of x [tokens, heads, D] is turned by the
    angle positions[t] * inv_freq[i].  Angle and rotation in float64 from the fp32 table, one rounding
    to the input dtype."""
    half = x.shape[-1] // 2
    ang = positions.double()[:, None] * inv_freq.double()[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    xd = x.double()
    a, b = xd[..., :half], xd[..., half:]
    return torch.cat((a * cos - b * sin, b * cos + a * sin), dim=-1).to(x.dtype)


def qk_norm_rope(x: torch.Tensor, weight: torch.Tensor, eps: float, positions: torch.Tensor,
                 inv_freq: torch.Tensor) -> torch.Tensor:
    """Per-head RMSNorm (as `rmsnorm`: the normalised value rounded to the input dtype, then the weight)
    followed by `rotate_half_rope` -- the Qwen3 q/k path in front of the attention (model wiring
    simple_rl.py:320-338: qk_norm, head_dim 128)."""
    return rotate_half_rope(rmsnorm(x, weight, eps), positions, inv_freq)


def argmax_lowest_index(x: torch.Tensor) -> torch.Tensor:
    """Index of the largest element of each row, ties to the LOWEST index, NaNs never selected
    (a row of NaNs gives 0).  Brute force over the row in Python order for small inputs is
    `max(range(n), key=lambda i: (x[i], -i))`; this is the vectorised form."""
    xf = x.float()
    xf = torch.where(torch.isnan(xf), torch.full_like(xf, float("-inf")), xf)
    m = xf.max(dim=-1, keepdim=True).values
    idx = torch.arange(x.shape[-1]).expand_as(xf)
    big = torch.full_like(idx, x.shape[-1])
    return torch.where(xf == m, idx, big).min(dim=-1).values


def decoder_prefill_logits(weights: dict, prompt: Sequence[int], num_q_heads: int, num_kv_heads: int, head_dim: int,
                           rms_eps: float, rope_theta: float, leaf: int = LEAF_BF16) -> torch.Tensor:
    """Last-token logits of a Qwen3-architecture decoder on one prompt, composed from the per-op oracles above with
    a rounding to bf16 wherever the kernels round (every op boundary): embedding -> [RMSNorm -> qkv (single
    accumulator mm) -> per-head q/k RMSNorm + rotary -> causal attention -> o_proj (tree matmul) -> add + RMSNorm ->
    gate_up (mm) -> SiLU * up -> down_proj (tree matmul)] x layers -> add + RMSNorm -> lm_head (mm).
    Model wiring as the reference's harness uses it (simple_rl.py:320-338: qk_norm, head_dim, GQA); the row-split
    layers are the patched RowParallelLinear forward (src/patch/patch_tp_invariant.py:11-46).

    `weights`: CPU bf16 tensors: embed [V,H], lm_head [V,H], final_norm [H], layers = list of dicts with
    input_norm, post_norm [H], q_norm, k_norm [D], qkv_w [(Hq+2Hkv)D, H], gate_up_w [2I, H], o_w [H, Hq*D],
    down_w [H, I].
    """
    Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
    tok = torch.tensor(list(prompt), dtype=torch.long)
    pos = torch.arange(len(prompt))
    inv = rope_inv_freq(D, rope_theta)
    x = weights["embed"][tok]
    residual = None
    for lw in weights["layers"]:
        if residual is None:
            residual = x
            h = rmsnorm(x, lw["input_norm"], rms_eps)
        else:
            h, residual = rmsnorm(x, lw["input_norm"], rms_eps, residual=residual)
        qkv = matmul_single_acc(h, lw["qkv_w"].t())
        q = qk_norm_rope(qkv[:, : Hq * D].reshape(-1, Hq, D), lw["q_norm"], rms_eps, pos, inv)
        k = qk_norm_rope(qkv[:, Hq * D: (Hq + Hkv) * D].reshape(-1, Hkv, D), lw["k_norm"], rms_eps, pos, inv)
        v = qkv[:, (Hq + Hkv) * D:].reshape(-1, Hkv, D)
        att = causal_attention(q, k, v, 1.0 / math.sqrt(D)).to(torch.bfloat16).reshape(-1, Hq * D)
        x = matmul_tree(att, lw["o_w"].t(), leaf=leaf)
        h, residual = rmsnorm(x, lw["post_norm"], rms_eps, residual=residual)
        act = silu_mul(matmul_single_acc(h, lw["gate_up_w"].t()))
        x = matmul_tree(act, lw["down_w"].t(), leaf=leaf)
    h, _ = rmsnorm(x, weights["final_norm"], rms_eps, residual=residual)
    return matmul_single_acc(h[-1:], weights["lm_head"].t())[0]


# --------------------------------------------------------------------------------------------
# seeded synthetic inputs shared by the tests, the smoke check and the benchmark
# --------------------------------------------------------------------------------------------
def gaussian_bf16(shape, std: float, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


def silu_gated_bf16(shape, seed: int) -> torch.Tensor:
    """Activation of a SiLU-gated MLP: g1 * silu(g2) with g1, g2 ~ N(0,1), rounded to bf16."""
    g = torch.Generator().manual_seed(seed)
    g1 = torch.randn(shape, generator=g, dtype=torch.float32)
    g2 = torch.randn(shape, generator=g, dtype=torch.float32)
    return (g1 * torch.nn.functional.silu(g2)).to(torch.bfloat16)


def integer_bf16(shape, lo: int, hi: int, seed: int) -> torch.Tensor:
    """Uniform integers in [lo, hi]: every chunk sum is an integer, exact in fp32 in any order."""
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).to(torch.bfloat16)


def bf16_ulp_distance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in units of bf16 representable values (sign-magnitude order), elementwise."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
        return torch.where(i >= 0x8000, 0x8000 - i, i)
    return (key(a) - key(b)).abs()


def outside_tolerance(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Mask of elements that violate the stated tolerance for random inputs: more than 1 bf16 ulp from the
    oracle AND more than 2^-8 of the output scale (max |want|) away in absolute terms."""
    got, want = got.cpu(), want.cpu()
    scale = want.float().abs().max()
    return (bf16_ulp_distance(got, want) > 1) & ((got.float() - want.float()).abs() > 2.0 ** -8 * scale)
