// Tree-ordered bf16 GEMM for gfx950, large-M path: 128x256 output tile per work-group, 8 wavefronts
// (2 per SIMD) of 64x64 each, K staged through LDS in 64-element slices.
//
// Same arithmetic contract as gemm_tiled.hip (and therefore the same bits): per leaf a chain of
// 16x16x32 bf16 MFMAs over k in ascending order into a zeroed fp32 accumulator, one rounding to bf16,
// then the binary-counter merge (level 0 left-to-right over FLB leaves, adjacent pairs above), every
// node rounded to bf16.  Replaces matmul_kernel_tp_persistent, src/tbik/tree_based_matmul.py:50-187.
//
// What differs is where the partials live and when the merge runs:
//   * only the running level-0 sum and the first binary level stay in registers; deeper levels are
//     parked in a global workspace (each lane reads back exactly the bytes it wrote, 16 B per lane,
//     fully coalesced).  They are touched once per 2, 4, 8 ... groups, so the traffic is a few percent
//     of the operand traffic, and the register file keeps room for two waves per SIMD.
//   * the merge of leaf j is deferred into leaf j+1: the finished accumulator is only packed to bf16
//     (which frees it for the next leaf's first MFMA), and a quarter of the tiles is merged in each of
//     the next leaf's K slices, so the VALU work rides in the shadow of the MFMAs.
#include "common.h"

namespace tbik {

struct WideArgs {
  const uint16_t* X;   // [M,K], row stride ldx
  const uint16_t* W;   // [N,K], row stride ldw
  uint16_t* C;         // [M,N], row stride ldc
  const uint16_t* bias;
  u32x4* ws;           // parked tree levels: [level][tile][wave][chunk 0..7][lane]
  int64_t ldx, ldw, ldc;
  int M, N, K;
  int T, flb, lb;
  int vec_store;
};

namespace wide {
constexpr int BM = 128, BN = 256, BK = 64;
constexpr int NT = 512;
constexpr int TM = 4, TN = 4;             // 16x16 MFMA tiles per wave: 64x64
constexpr int STAGE = (BM + BN) * BK;     // bf16 elements per LDS stage
constexpr int XCH = BM * 8 / NT;          // 16-byte chunks per thread per stage: 2
constexpr int WCH = BN * 8 / NT;          // 4
constexpr int RL = 1;                     // binary levels kept in registers
constexpr int NTILE = TM * TN;            // 16 tiles, each 2 packed registers per lane
constexpr int MAXLB = 12;

__device__ __forceinline__ int lds_off(int r, int c) { return r * BK + ((c ^ (r & 7)) << 3); }
}  // namespace wide

size_t wide_workspace_bytes(int M, int N, int lb) {
  using namespace wide;
  if (lb <= RL) return 0;
  const size_t tiles = (size_t)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  return (size_t)(lb - RL) * tiles * (NT / 64) * 8 * 64 * sizeof(u32x4);
}

template <int LS>
__global__ __launch_bounds__(wide::NT) void gemm_tree_wide_kernel(const WideArgs p) {
  using namespace wide;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 2;  // 0..1
  const int wn = wave & 3;   // 0..3

  const int tiles_m = (p.M + BM - 1) / BM;
  const int tiles_n = (p.N + BN - 1) / BN;
  int lid = blockIdx.x;
  {
    const int nwg = gridDim.x;
    if ((nwg & 7) == 0) lid = (lid & 7) * (nwg >> 3) + (lid >> 3);  // consecutive ids share an XCD
  }
  constexpr int GROUP = 4;
  const int per_group = GROUP * tiles_n;
  const int group_id = lid / per_group;
  const int first_m = group_id * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int pid_m = first_m + (lid % per_group) % gsz;
  const int pid_n = (lid % per_group) / gsz;
  const int m0 = pid_m * BM;
  const int n0 = pid_n * BN;
  const int tile_id = pid_m * tiles_n + pid_n;
  const int ntiles = tiles_m * tiles_n;

  // ---- global -> register -> LDS staging
  const uint16_t* xptr[XCH];
  const uint16_t* wptr[WCH];
  int xdst[XCH], wdst[WCH];
#pragma unroll
  for (int i = 0; i < XCH; i++) {
    const int q = tid + i * NT;
    const int r = q >> 3, c = q & 7;
    xptr[i] = p.X + (int64_t)min(m0 + r, p.M - 1) * p.ldx + c * 8;
    xdst[i] = lds_off(r, c);
  }
#pragma unroll
  for (int i = 0; i < WCH; i++) {
    const int q = tid + i * NT;
    const int r = q >> 3, c = q & 7;
    wptr[i] = p.W + (int64_t)min(n0 + r, p.N - 1) * p.ldw + c * 8;
    wdst[i] = BM * BK + lds_off(r, c);
  }
  u32x4 xreg[XCH], wreg[WCH];
  auto load_stage = [&](int s) __attribute__((always_inline)) {
    const int k0 = s * BK;
#pragma unroll
    for (int i = 0; i < XCH; i++) xreg[i] = *reinterpret_cast<const u32x4*>(xptr[i] + k0);
#pragma unroll
    for (int i = 0; i < WCH; i++) wreg[i] = *reinterpret_cast<const u32x4*>(wptr[i] + k0);
  };
  auto store_stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < XCH; i++) *reinterpret_cast<u32x4*>(smem + buf * STAGE + xdst[i]) = xreg[i];
#pragma unroll
    for (int i = 0; i < WCH; i++) *reinterpret_cast<u32x4*>(smem + buf * STAGE + wdst[i]) = wreg[i];
  };

  const int frow = lane & 15;
  const int fchk = lane >> 4;

  f32x4 acc[TM][TN];
  uint32_t t[NTILE][2];    // packed leaf waiting to be merged (leaf j while leaf j+1 is computed)
  uint32_t s0[NTILE][2];   // level 0 running sum
  uint32_t sb0[NTILE][2];  // first binary level
  // merge state of the leaf held in t (uniform over the block)
  int c0 = 0;  // leaves already absorbed at level 0 before that leaf
  int g = 0;   // groups completed before that leaf

  // parked levels: level l >= RL, this wave's 8 chunks of 16 B per lane
  auto ws_ptr = [&](int l, int chunk) __attribute__((always_inline)) -> u32x4* {
    return p.ws + ((((int64_t)(l - RL) * ntiles + tile_id) * (NT / 64) + wave) * 8 + chunk) * 64 + lane;
  };

  // Merge tiles [4q, 4q+4) of the leaf in t into the stack; returns with t = the node that left the stack
  // when the whole tree completed (only meaningful for the last leaf).
  auto merge_quarter = [&](int q) __attribute__((always_inline)) {
    if (c0 != 0) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        t[4 * q + i][0] = add_bf16x2(s0[4 * q + i][0], t[4 * q + i][0]);
        t[4 * q + i][1] = add_bf16x2(s0[4 * q + i][1], t[4 * q + i][1]);
      }
    }
    if (c0 + 1 == p.flb) {
      bool parked = false;
      if (p.lb > 0) {
        if (g & 1) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            t[4 * q + i][0] = add_bf16x2(sb0[4 * q + i][0], t[4 * q + i][0]);
            t[4 * q + i][1] = add_bf16x2(sb0[4 * q + i][1], t[4 * q + i][1]);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            sb0[4 * q + i][0] = t[4 * q + i][0];
            sb0[4 * q + i][1] = t[4 * q + i][1];
          }
          parked = true;
        }
      }
      for (int l = RL; l < p.lb && !parked; l++) {
        u32x4* w0 = ws_ptr(l, 2 * q);
        u32x4* w1 = ws_ptr(l, 2 * q + 1);
        if ((g >> l) & 1) {
          const u32x4 a = *w0, b = *w1;
          t[4 * q + 0][0] = add_bf16x2(a[0], t[4 * q + 0][0]);
          t[4 * q + 0][1] = add_bf16x2(a[1], t[4 * q + 0][1]);
          t[4 * q + 1][0] = add_bf16x2(a[2], t[4 * q + 1][0]);
          t[4 * q + 1][1] = add_bf16x2(a[3], t[4 * q + 1][1]);
          t[4 * q + 2][0] = add_bf16x2(b[0], t[4 * q + 2][0]);
          t[4 * q + 2][1] = add_bf16x2(b[1], t[4 * q + 2][1]);
          t[4 * q + 3][0] = add_bf16x2(b[2], t[4 * q + 3][0]);
          t[4 * q + 3][1] = add_bf16x2(b[3], t[4 * q + 3][1]);
        } else {
          *w0 = u32x4{t[4 * q + 0][0], t[4 * q + 0][1], t[4 * q + 1][0], t[4 * q + 1][1]};
          *w1 = u32x4{t[4 * q + 2][0], t[4 * q + 2][1], t[4 * q + 3][0], t[4 * q + 3][1]};
          parked = true;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        s0[4 * q + i][0] = t[4 * q + i][0];
        s0[4 * q + i][1] = t[4 * q + i][1];
      }
    }
  };
  auto advance_counters = [&]() __attribute__((always_inline)) {
    if (c0 + 1 == p.flb) {
      c0 = 0;
      g++;
    } else {
      c0++;
    }
  };

  const int nstages = p.T * LS;
  load_stage(0);
  store_stage(0);
  __syncthreads();

  for (int j = 0; j < p.T; j++) {
#pragma unroll
    for (int i = 0; i < LS; i++) {
      const int s = j * LS + i;
      load_stage(min(s + 1, nstages - 1));
      const uint16_t* bx = smem + (s & 1) * STAGE;
      const uint16_t* bw = bx + BM * BK;
#pragma unroll
      for (int kk = 0; kk < 2; kk++) {
        bf16x8 fx[TM], fw[TN];
#pragma unroll
        for (int a = 0; a < TM; a++) fx[a] = *reinterpret_cast<const bf16x8*>(bx + lds_off((wm * TM + a) * 16 + frow, kk * 4 + fchk));
#pragma unroll
        for (int b = 0; b < TN; b++) fw[b] = *reinterpret_cast<const bf16x8*>(bw + lds_off((wn * TN + b) * 16 + frow, kk * 4 + fchk));
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
          for (int b = 0; b < TN; b++) {
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[b], fx[a], (i == 0 && kk == 0) ? zero : acc[a][b], 0, 0, 0);
          }
      }
      // deferred merge of the previous leaf: a quarter (LS == 4) or a half (LS == 2) per K slice
      if (j > 0) {
#pragma unroll
        for (int q = i * (4 / LS); q < (i + 1) * (4 / LS); q++) merge_quarter(q);
      }
      store_stage((s + 1) & 1);
      __syncthreads();
    }
    if (j > 0) advance_counters();
    // the finished leaf: round once to bf16; the accumulator is free again
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++) {
        t[a * TN + b][0] = pack_bf16x2(acc[a][b][0], acc[a][b][1]);
        t[a * TN + b][1] = pack_bf16x2(acc[a][b][2], acc[a][b][3]);
      }
  }
  // merge of the last leaf: every level carries, t ends as the root
#pragma unroll
  for (int q = 0; q < 4; q++) merge_quarter(q);

  // ---- store
#pragma unroll
  for (int a = 0; a < TM; a++) {
    const int m = m0 + (wm * TM + a) * 16 + frow;
#pragma unroll
    for (int b = 0; b < TN; b++) {
      const int n = n0 + (wn * TN + b) * 16 + fchk * 4;
      if (m >= p.M || n >= p.N) continue;
      uint32_t lo = t[a * TN + b][0], hi = t[a * TN + b][1];
      if (p.bias) {
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < p.N) bv[e] = bf16_bits_to_f32(p.bias[n + e]);
        lo = add_bf16x2(lo, pack_bf16x2(bv[0], bv[1]));
        hi = add_bf16x2(hi, pack_bf16x2(bv[2], bv[3]));
      }
      uint16_t* dst = p.C + (int64_t)m * p.ldc + n;
      if (p.vec_store && n + 3 < p.N) {
        *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
      } else {
        const uint16_t v[4] = {(uint16_t)(lo & 0xffff), (uint16_t)(lo >> 16), (uint16_t)(hi & 0xffff), (uint16_t)(hi >> 16)};
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < p.N) dst[e] = v[e];
      }
    }
  }
}

int gemm_tree_wide_launch(const WideArgs& a, int leaf_k, hipStream_t stream) {
  using namespace wide;
  constexpr size_t smem = (size_t)2 * STAGE * sizeof(uint16_t);  // 96 KiB
  const int64_t tiles = (int64_t)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  if (tiles <= 0 || tiles > 0x7fffffff || a.lb > MAXLB) return TBIK_ERR_UNSUPPORTED;
  if (leaf_k == 256) {
    auto kern = gemm_tree_wide_kernel<4>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return hip_code(e);
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(NT), smem, stream, a);
  } else if (leaf_k == 128) {
    auto kern = gemm_tree_wide_kernel<2>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return hip_code(e);
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(NT), smem, stream, a);
  } else {
    return TBIK_ERR_UNSUPPORTED;
  }
  return hip_code(hipGetLastError());
}

}  // namespace tbik
