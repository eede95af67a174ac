// fp32 GEMM for gfx950 with the same two accumulation disciplines as the 16-bit kernels:
//
//   TREE = true   tree-ordered (TP-invariant) matmul, the float32 branch of the reference's dtype-keyed
//                 configuration (leaf 128, src/tbik/tree_based_matmul.py:223-231): a leaf is the fp32 sum of its
//                 128 products, leaves merge through the binary counter (level 0 left to right over FLB leaves,
//                 adjacent pairs above), every node one fp32 addition.
//   TREE = false  one fp32 accumulator over all of K (aten::mm / aten::addmm on fp32 tensors in batch-invariant
//                 mode, src/bio/batch_invariant_ops.py:127-197).
//
// Products run on v_mfma_f32_16x16x4_f32 (full fp32 inputs; the reference's Triton dot uses TF32 on its hardware,
// so parity with it is to tolerance only).  K is walked in chunks of 16: a lane loads four consecutive k of its
// row (16 bytes) and the chunk's four MFMAs take k = 4g + j (g = lane / 16) -- a fixed permutation of the chunk,
// so the summation order of an element is a function of K alone: row m never sees M, tiles or the launch.
// This is a correctness path (fp32 matmuls are rare in the models the reference serves): operands are read
// straight from global memory, 64x64 tile per work-group, 4 waves of 32x32.
#include "common.h"

namespace tbik {

struct GemmF32Args {
  const float* X;  // [M,K], row stride ldx
  const float* W;  // [N,K], row stride ldw
  float* C;        // [M,N], row stride ldc
  const float* bias;
  int64_t ldx, ldw, ldc;
  int M, N, K;
  int T, flb, lb;  // leaves of 128, leaves per level-0 group, binary levels (TREE)
};

constexpr int F32_LBMAX = 8;

template <bool TREE>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const GemmF32Args p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.N + 63) / 64;
  const int m0 = (blockIdx.x / tiles_n) * 64 + wm * 32;
  const int n0 = (blockIdx.x % tiles_n) * 64 + wn * 32;
  const int r16 = lane & 15, g = lane >> 4;

  const float* xp[2];
  const float* wp[2];
#pragma unroll
  for (int a = 0; a < 2; a++) xp[a] = p.X + (int64_t)min(m0 + a * 16 + r16, p.M - 1) * p.ldx + 4 * g;
#pragma unroll
  for (int b = 0; b < 2; b++) wp[b] = p.W + (int64_t)min(n0 + b * 16 + r16, p.N - 1) * p.ldw + 4 * g;

  f32x4 acc[2][2];
  f32x4 s0[2][2], sb[F32_LBMAX][2][2];
  int c0 = 0, grp = 0;
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++) acc[a][b] = zero;

  const int nchunks = p.K / 16;
  const int per_leaf = TREE ? 8 : nchunks;
  const int nleaves = TREE ? p.T : 1;
  int chunk = 0;
  for (int j = 0; j < nleaves; j++) {
    for (int i = 0; i < per_leaf; i++, chunk++) {
      f32x4 fx[2], fw[2];
#pragma unroll
      for (int a = 0; a < 2; a++) fx[a] = *reinterpret_cast<const f32x4*>(xp[a] + (int64_t)chunk * 16);
#pragma unroll
      for (int b = 0; b < 2; b++) fw[b] = *reinterpret_cast<const f32x4*>(wp[b] + (int64_t)chunk * 16);
#pragma unroll
      for (int e = 0; e < 4; e++)
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int b = 0; b < 2; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(fw[b][e], fx[a][e], acc[a][b], 0, 0, 0);
    }
    if (!TREE) break;
    // leaf done: binary-counter merge in fp32 (all conditions are uniform over the block)
    f32x4 t[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int b = 0; b < 2; b++) {
        t[a][b] = c0 != 0 ? s0[a][b] + acc[a][b] : acc[a][b];
        acc[a][b] = zero;
      }
    c0++;
    if (c0 == p.flb) {
      c0 = 0;
      bool parked = false;
#pragma unroll
      for (int l = 0; l < F32_LBMAX; l++) {
        if (!parked && l < p.lb) {
          if ((grp >> l) & 1) {
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
              for (int b = 0; b < 2; b++) t[a][b] = sb[l][a][b] + t[a][b];
          } else {
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
              for (int b = 0; b < 2; b++) sb[l][a][b] = t[a][b];
            parked = true;
          }
        }
      }
      grp++;
      if (j == nleaves - 1) {
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int b = 0; b < 2; b++) acc[a][b] = t[a][b];  // the root
      }
    } else {
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) s0[a][b] = t[a][b];
    }
  }

#pragma unroll
  for (int a = 0; a < 2; a++) {
    const int m = m0 + a * 16 + r16;
#pragma unroll
    for (int b = 0; b < 2; b++) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int n = n0 + b * 16 + 4 * g + e;
        if (m < p.M && n < p.N) p.C[(int64_t)m * p.ldc + n] = acc[a][b][e] + (p.bias ? p.bias[n] : 0.f);
      }
    }
  }
}

int gemm_f32_dispatch(bool tree, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                      int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, hipStream_t stream) {
  if (M < 0 || N < 0 || K <= 0) return TBIK_ERR_INVALID;
  if (M == 0 || N == 0) return TBIK_OK;
  if (!A || !B || !C) return TBIK_ERR_INVALID;
  if (ldb_k != 1) return TBIK_ERR_UNSUPPORTED;  // row-major [K,N] weights are repacked by the caller
  if (lda < K || ldb_n < K || ldc < N) return TBIK_ERR_INVALID;
  auto mis = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) != 0; };
  if (mis(A) || mis(B) || (lda & 3) || (ldb_n & 3) || (K & 15)) return TBIK_ERR_ALIGNMENT;
  if (reinterpret_cast<uintptr_t>(C) & 3) return TBIK_ERR_ALIGNMENT;
  GemmF32Args a{static_cast<const float*>(A), static_cast<const float*>(B), static_cast<float*>(C),
                static_cast<const float*>(bias), lda, ldb_n, ldc, M, N, K, 0, 1, 0};
  const int64_t tiles = (int64_t)((M + 63) / 64) * ((N + 63) / 64);
  if (tiles > 0x7fffffff) return TBIK_ERR_INVALID;
  if (tree) {
    if (leaf_k != 128) return TBIK_ERR_UNSUPPORTED;
    int T, flb, level_k;
    if (tbik_tree_params(K, leaf_k, &T, &flb, &level_k) != TBIK_OK) return TBIK_ERR_INVALID;
    if (level_k - 1 > F32_LBMAX) return TBIK_ERR_UNSUPPORTED;
    a.T = T;
    a.flb = flb;
    a.lb = level_k - 1;
    hipLaunchKernelGGL(gemm_f32_kernel<true>, dim3((unsigned)tiles), dim3(256), 0, stream, a);
  } else {
    hipLaunchKernelGGL(gemm_f32_kernel<false>, dim3((unsigned)tiles), dim3(256), 0, stream, a);
  }
  return hip_code(hipGetLastError());
}

}  // namespace tbik
