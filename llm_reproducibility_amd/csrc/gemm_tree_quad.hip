// Tree-ordered bf16 GEMM for gfx950, path of 64 .. 512 rows with short K shards: 128x128 tiles, 4 wavefronts (one per
// SIMD) of 64x64 each, K streamed through a 4-slot LDS ring in 64-element slices -- the pipeline of
// gemm_single_acc_quad.hip with the merge tree of gemm_tree_wide.hip, and the whole tree of a shard in registers.
// Replaces matmul_kernel_tp_persistent, src/tbik/tree_based_matmul.py:50-187, where one row of 128x256 tiles needs a
// cut of K into sixteen shards (and a pass over sixteen partial results) to occupy the chip: with tiles half as wide
// eight shards do.  Per element the arithmetic is that of every other tree kernel of this library (one chain of
// 16x16x32 MFMAs per leaf over k ascending, one rounding per leaf, a left-to-right sum over the leaves of a group, an
// adjacent-pair tree over the groups, every node rounded to bf16), so the bits are the same.
//
// A wave's tile is 64x64: 32 packed registers per tree level, so the running sum, the pending leaf and one binary level
// (shards of at most two groups of leaves) sit next to the accumulators without a workspace.  The finished leaf j is
// rounded into the pending registers and merged while leaf j+1 multiplies; with one wave per SIMD nothing else hides
// that work, so it is cut into pieces of two or three instructions, each behind one MFMA (an MFMA occupies the matrix
// pipe for 16 cycles and the wave issues in order: a run of vector instructions leaves the pipe idle).  How a leaf
// merges (it opens a group, joins the running sum, or closes a group) is fixed per leaf, so there is one straight-line
// loop body per kind.
//
// Where it pays (measured on MI355X against the 128x256-tile kernels with their own best split, weights cold): only
// where a work-group's shard is short, 512 .. 1536 of K -- [128,4096]x[4096,4096] 20.3 -> 17.7 us, [128,6144]x[6144,4096]
// 25.1 -> 20.7, [128,12288]x[12288,4096] 33.8 -> 32.1, [96,6144]x[6144,3072] 22.4 -> 18.8, [64,8192]x[8192,4096] 22.9 -> 21.0, [256,6144]x[6144,2048] 23.6 -> 19.9.  On longer shards a slice
// costs 0.59 us against 0.385 us in the single-accumulator kernel with the same tile: the tree's two to three vector
// instructions per MFMA do not fit behind the MFMAs of ONE wave per SIMD ([512,8192]x[8192,5120] uncut on 128x96 tiles
// 75 us against 70 us for the 128x256-tile kernels with their K split; [256,K]x[K,N] 10-20 % slower from K = 6144 on),
// which is why the tile widths of 32, 64 and 96 columns, the deeper rings and the leaves of 128 that this pipeline
// also allows were measured and are not built.
#include <type_traits>

#include "common.h"
#include "gemm_args.h"
#include "lds_direct.h"

namespace tbik {

namespace tq {
constexpr int BM = 128, BK = 64, NT = 256, NWAVE = 4, TM = 4;
constexpr int XDMA = BM / 8 / NWAVE;  // direct loads of X rows per wave per slice: 4 (8 rows of 128 B each)
constexpr int MAXL = 1;               // binary levels of a shard's tree (all in registers)
template <int TN>
struct Shape {
  static constexpr int BN = 2 * TN * 16;  // two waves across N, TN MFMA tiles each
  static constexpr int ROWS = BM + BN;
  static constexpr int STAGE_BYTES = ROWS * BK * 2;
  static constexpr int NDMA = ROWS / 8 / NWAVE;
};
enum Kind { K_FIRST = 0, K_ADD = 1, K_CARRY = 2 };  // the pending leaf opens a group / joins the running sum / closes the group
}  // namespace tq

// TN: 16-column MFMA tiles per wave (4: the 128-column tile).  LS: slices per leaf (4: leaves of 256).  NSLOT: slices of
// the ring.
template <int TN, int NSLOT, int LS>
__global__ __launch_bounds__(tq::NT) void gemm_tree_quad_kernel(const WideArgs p) {
  using namespace tq;
  static_assert(NSLOT >= 3 && TN >= 1 && TN <= 4, "tile shape");
  constexpr int BN = Shape<TN>::BN, STAGE_BYTES = Shape<TN>::STAGE_BYTES, NDMA = Shape<TN>::NDMA;
  constexpr int NREG = TM * TN * 2;  // packed bf16 pairs per lane per tree level
  constexpr int G = LS * 8;          // groups of TN MFMAs per leaf: the merge of the pending leaf is spread over them
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int shard = blockIdx.y;

  const int tiles_m = (p.M + BM - 1) / BM;
  const int tiles_n = (p.N + BN - 1) / BN;
  int lid = blockIdx.x;
  {
    const int nwg = gridDim.x;
    lid = xcd_contiguous_tile(lid, nwg);
  }
  constexpr int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int group_id = lid / per_group;
  const int first_m = group_id * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int pid_m = first_m + (lid % per_group) % gsz;
  const int pid_n = (lid % per_group) / gsz;
  const int m0 = pid_m * BM, n0 = pid_n * BN;

  const uint8_t* xbase = reinterpret_cast<const uint8_t*>(p.X + (int64_t)m0 * p.ldx + shard * p.k_shard);
  const uint8_t* wbase = reinterpret_cast<const uint8_t*>(p.W + (int64_t)n0 * p.ldw + shard * p.k_shard);
  uint32_t voff[NDMA];
  {
    const int r = lane >> 3, c = (lane & 7) ^ r;
#pragma unroll
    for (int i = 0; i < NDMA; i++) {
      const int row = (i * NWAVE + wave) * 8 + r;  // X rows, then W rows; rows past the edge are clamped
      if (i < XDMA) voff[i] = (uint32_t)(((min(m0 + row, p.M - 1) - m0) * p.ldx + c * 8) * 2);
      else voff[i] = (uint32_t)(((min(n0 + row - BM, p.N - 1) - n0) * p.ldw + c * 8) * 2);
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int nstages = p.T * LS;
  auto dma_one = [&](int s, int slot, int i) __attribute__((always_inline)) {
    const uint8_t* b = (i < XDMA ? xbase : wbase) + (int64_t)min(s, nstages - 1) * (BK * 2);
    dma16(lds0 + slot * STAGE_BYTES + (i * NWAVE + wave) * 1024, voff[i], b);
  };
  const int frow = lane & 15, fchk = lane >> 4;
  const uint32_t xfrag = ((wm * TM * 16 + frow) * BK + ((fchk ^ (frow & 7)) << 3)) * 2;
  const uint32_t wfrag = (BM * BK + (wn * TN * 16 + frow) * BK + ((fchk ^ (frow & 7)) << 3)) * 2;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 fx[2][TM], fw[2][TN];
  auto read_x = [&](int buf, int slot, int kk, int a) __attribute__((always_inline)) {
    fx[buf][a] = *reinterpret_cast<const bf16x8*>(smem + slot * STAGE_BYTES + (xfrag ^ (kk * 64)) + a * 16 * BK * 2);
  };
  auto read_w = [&](int buf, int slot, int kk, int b) __attribute__((always_inline)) {
    fw[buf][b] = *reinterpret_cast<const bf16x8*>(smem + slot * STAGE_BYTES + (wfrag ^ (kk * 64)) + b * 16 * BK * 2);
  };

  // tree state, packed bf16 pairs: register (a * TN + b) * 2 + h holds elements 2h, 2h+1 of MFMA tile (a, b)
  uint32_t t[NREG];         // the finished leaf that waits for its merge (leaf j while leaf j+1 multiplies)
  uint32_t s0[NREG];        // running sum of the current group
  uint32_t lv[MAXL][NREG];  // binary levels
#pragma unroll
  for (int r = 0; r < NREG; r++) {
    t[r] = 0;
    s0[r] = 0;
#pragma unroll
    for (int l = 0; l < MAXL; l++) lv[l][r] = 0;
  }

  // prologue: NSLOT slices in flight, slice 0 visible, fragments of the first k step loaded
#pragma unroll
  for (int s = 0; s < NSLOT; s++)
#pragma unroll
    for (int i = 0; i < NDMA; i++) dma_one(s, s, i);
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSLOT - 1) * NDMA) : "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int a = 0; a < TM; a++) read_x(0, 0, 0, a);
#pragma unroll
  for (int b = 0; b < TN; b++) read_w(0, 0, 0, b);

  int slot = 0;
  // One leaf (LS slices).  KIND says how the PENDING leaf (in t) is merged meanwhile.  Group gi of the leaf's G groups of
  // MFMAs merges the registers [gi * NREG / G, (gi + 1) * NREG / G); the rows of the leaf that is being computed are
  // rounded into t one group behind the row's last MFMA -- rows 0..2 in the last k step, row 3 in the first group of the
  // next leaf -- always after the merge has consumed those registers of the leaf before.
  auto leaf_body = [&](auto kind_c, int j) __attribute__((always_inline)) {
    constexpr int KIND = decltype(kind_c)::value;
    constexpr int NPIECE = KIND == K_FIRST ? 1 : 3;
#pragma unroll
    for (int i = 0; i < LS; i++) {
      const int s = j * LS + i;
      const int nslot = slot + 1 == NSLOT ? 0 : slot + 1;
      const int pslot = slot == 0 ? NSLOT - 1 : slot - 1;
#pragma unroll
      for (int kk = 0; kk < 2; kk++) {
        constexpr int NG = 4;
        constexpr int H1 = (NDMA + 1) / 2, H2 = NDMA - H1;
        static_assert(H1 <= NG && TM + TN <= 2 * NG, "schedule does not fit the groups");
#pragma unroll
        for (int q = 0; q < NG; q++) {
          const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
          const int rslot = kk == 0 ? slot : nslot;
          const int gi = i * 8 + kk * 4 + q;
          const int r0 = gi * NREG / G, r1 = (gi + 1) * NREG / G;
          float xl[2], xh[2], yl[2], yh[2];
          uint32_t v[2];
          // piece `pc` of the merge of this group's registers
          auto piece = [&](int pc) __attribute__((always_inline)) {
#pragma unroll
            for (int r = r0; r < r1; r++) {
              const int u = r - r0;
              if (KIND == K_FIRST) {
                if (pc == 0) s0[r] = t[r];
              } else {
                if (pc == 0) {
                  xl[u] = bf16_lo(t[r]);
                  xh[u] = bf16_hi(t[r]);
                } else if (pc == 1) {
                  yl[u] = bf16_lo(s0[r]);
                  yh[u] = bf16_hi(s0[r]);
                } else if (pc == 2) {
                  v[u] = pack_bf16x2(yl[u] + xl[u], yh[u] + xh[u]);
                  if (KIND == K_ADD) s0[r] = v[u];
                  if (KIND == K_CARRY) lv[0][r] = v[u];  // the first of the shard's two groups: level 0 is empty
                }
              }
            }
          };
          // what follows MFMA jj of the group: one fragment read or direct load, a piece of the merge, and in the last
          // k step of the leaf the rounding of one tile of the row before
          auto behind = [&](int jj) __attribute__((always_inline)) {
            if (jj < 2) {
              const int f = 2 * q + jj;
              if (f < TM) read_x(kk ^ 1, rslot, kk ^ 1, f);
              else if (f - TM < TN) read_w(kk ^ 1, rslot, kk ^ 1, f - TM);
            } else if (jj == 2) {
              if (kk == 1 && q < H1) dma_one(s + NSLOT, slot, q);
              if (kk == 0 && q < H2 && s > 0) dma_one(s + NSLOT - 1, pslot, H1 + q);
            }
            if (jj < TN) {
              // pieces beyond the group's MFMAs go behind the last one
              if (jj < TN - 1) {
                if (jj < NPIECE) piece(jj);
              } else {
#pragma unroll
                for (int pc = jj; pc < NPIECE; pc++) piece(pc);
              }
              int prow = -1;
              if (i == LS - 1 && kk == 1 && q >= 1) prow = q - 1;
              if (i == 0 && kk == 0 && q == 0) prow = TM - 1;  // of the leaf before (zeros in front of the first leaf)
              if (prow >= 0) {
                t[(prow * TN + jj) * 2] = pack_bf16x2(acc[prow][jj][0], acc[prow][jj][1]);
                t[(prow * TN + jj) * 2 + 1] = pack_bf16x2(acc[prow][jj][2], acc[prow][jj][3]);
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          };
#pragma unroll
          for (int jj = 0; jj < TN; jj++) {
            acc[q][jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[kk][jj], fx[kk][q], (i == 0 && kk == 0) ? zero : acc[q][jj], 0, 0, 0);
            behind(jj);
          }
#pragma unroll
          for (int jj = TN; jj < 3; jj++) behind(jj);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (kk == 0) {
          // mid-slice: slice s+1 has landed (this wave's share) and every fragment read of slice s is done
          asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NSLOT - 2) * NDMA) : "memory");
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
      }
      slot = nslot;
    }
  };

  int kind = K_FIRST;  // in front of the first leaf the pending registers hold zeros: they "open a group" harmlessly
  int c0 = 0;          // leaves of the current group that are merged or pending
  for (int j = 0; j < p.T; j++) {
    switch (kind) {
      case K_FIRST: leaf_body(std::integral_constant<int, K_FIRST>{}, j); break;
      case K_ADD: leaf_body(std::integral_constant<int, K_ADD>{}, j); break;
      default: leaf_body(std::integral_constant<int, K_CARRY>{}, j); break;
    }
    if (j == p.T - 1) break;  // the last leaf is merged below
    // leaf j is (but for its last row) in the pending registers: how it merges
    if (c0 == 0 && p.flb > 1) {
      kind = K_FIRST;
      c0 = 1;
    } else if (c0 + 1 < p.flb) {
      kind = K_ADD;
      c0++;
    } else {
      kind = K_CARRY;  // never the last group here: with lb <= 1 it is the first of two, and its sum waits at level 0
      c0 = 0;
    }
  }

  // the last leaf: its last row, then every level carries and t ends as the root
#pragma unroll
  for (int b = 0; b < TN; b++) {
    t[((TM - 1) * TN + b) * 2] = pack_bf16x2(acc[TM - 1][b][0], acc[TM - 1][b][1]);
    t[((TM - 1) * TN + b) * 2 + 1] = pack_bf16x2(acc[TM - 1][b][2], acc[TM - 1][b][3]);
  }
  if (c0 != 0) {
#pragma unroll
    for (int r = 0; r < NREG; r++) t[r] = add_bf16x2(s0[r], t[r]);
  }
#pragma unroll
  for (int l = 0; l < MAXL; l++) {
    if (l < p.lb) {
#pragma unroll
      for (int r = 0; r < NREG; r++) t[r] = add_bf16x2(lv[l][r], t[r]);
    }
  }

#pragma unroll
  for (int a = 0; a < TM; a++) {
    const int m = m0 + (wm * TM + a) * 16 + frow;
#pragma unroll
    for (int b = 0; b < TN; b++) {
      const int n = n0 + (wn * TN + b) * 16 + fchk * 4;
      if (m >= p.M || n >= p.N) continue;
      uint32_t lo = t[(a * TN + b) * 2], hi = t[(a * TN + b) * 2 + 1];
      if (p.bias) {
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < p.N) bv[e] = bf16_bits_to_f32(p.bias[n + e]);
        lo = add_bf16x2(lo, pack_bf16x2(bv[0], bv[1]));
        hi = add_bf16x2(hi, pack_bf16x2(bv[2], bv[3]));
      }
      uint16_t* dst = p.C + shard * p.c_shard + (int64_t)m * p.ldc + n;
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

template <int TN, int NSLOT, int LS>
static int tq_launch(const WideArgs& a, int split, hipStream_t stream) {
  using namespace tq;
  constexpr int BN = Shape<TN>::BN;
  constexpr size_t smem = (size_t)NSLOT * Shape<TN>::STAGE_BYTES;
  static_assert(smem <= 160 * 1024 && (NSLOT - 1) * Shape<TN>::NDMA < 64, "ring does not fit the LDS or the wait counter");
  const int64_t tiles = (int64_t)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  if (tiles <= 0 || tiles > 0x7fffffff || split <= 0 || split > 65535) return TBIK_ERR_UNSUPPORTED;
  if (a.T <= 0 || a.K != a.T * LS * BK || a.lb < 0 || a.lb > MAXL || a.flb < 1) return TBIK_ERR_UNSUPPORTED;
  if (a.ldx >= (1 << 22) || a.ldw >= (1 << 22)) return TBIK_ERR_UNSUPPORTED;  // 32-bit in-tile byte offsets
  static std::atomic<uint64_t> done{0};
  hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_tree_quad_kernel<TN, NSLOT, LS>), (int)smem, done);
  if (e != hipSuccess) return hip_code(e);
  hipLaunchKernelGGL((gemm_tree_quad_kernel<TN, NSLOT, LS>), dim3((unsigned)tiles, (unsigned)split), dim3(NT), smem, stream, a);
  return hip_code(hipGetLastError());
}

// a ring of four slices (128 KiB): 2-5 % ahead of three on half of the shapes measured, level with it on the rest; five
// are no better than three
int gemm_tree_quad_launch(const WideArgs& a, int split, hipStream_t stream) { return tq_launch<4, 4, 4>(a, split, stream); }

}  // namespace tbik
