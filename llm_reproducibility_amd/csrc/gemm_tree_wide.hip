// Tree-ordered bf16 / fp16 GEMM for gfx950, large-M path: 128x256 output tile per work-group, 8 wavefronts
// (2 per SIMD) of 64x64 each, K streamed through a 3-slot LDS ring in 64-element slices.  Leaves of 256 or 128;
// trees of leaves of 256 that carry often run on the sibling kernel in gemm_tree_wide_deep.hip (same bits).
//
// Same arithmetic contract as gemm_tiled.hip (and therefore the same bits): per leaf a chain of
// 16x16x32 bf16 MFMAs over k in ascending order into a zeroed fp32 accumulator, one rounding to bf16,
// then the binary-counter merge (level 0 left-to-right over FLB leaves, adjacent pairs above), every
// node rounded to bf16.  Replaces matmul_kernel_tp_persistent, src/tbik/tree_based_matmul.py:50-187.
//
// How it is arranged for CDNA4:
//   * operands go global -> LDS directly (global_load_lds_dwordx4), two K slices ahead of the MFMAs;
//     a lane picks the global chunk that belongs at its (linear) LDS position, which realises the XOR
//     bank swizzle on the source side.  One barrier per slice.
//   * the running level-0 sum and the first binary level of the merge tree stay in registers as packed
//     bf16; deeper levels (touched once per 2, 4, ... groups) are parked in a global workspace, each
//     lane reading back exactly the 16-byte words it wrote.  The level that is popped most often is
//     brought back through the same direct global->LDS path one K slice ahead of its use.
//   * the merge of leaf j is deferred into leaf j+1: the finished accumulator is only packed to bf16
//     (which frees it for the next leaf's first MFMA); a quarter of the tiles is merged in each of the
//     next leaf's K slices.  The leaf body is instantiated once per merge kind so that every slice is
//     straight-line code and the VALU work can issue in the shadow of the MFMAs.
// Compiled with -structurizecfg-skip-uniform-regions: the switch between the leaf bodies is wave-uniform; structurized,
// it becomes a chain of flow blocks whose preambles copy every live array whether or not a body runs.
#include <type_traits>

#include "common.h"
#include "gemm_args.h"
#include "lds_direct.h"

namespace tbik {

namespace wide {
constexpr int BM = 128, BN = 256, BK = 64;
constexpr int NT = 512;
constexpr int TM = 4, TN = 4;                 // 16x16 MFMA tiles per wave: 64x64
constexpr int ROWS = BM + BN;                 // LDS rows per slice: X rows, then W rows
constexpr int STAGE_BYTES = ROWS * BK * 2;    // 48 KiB
constexpr int NSLOT = 3;
constexpr int NDMA = ROWS / 8 / (NT / 64);    // direct loads per wave per slice: 6 (8 rows of 128 B each)
constexpr int RL = 1;                         // binary levels kept in registers
constexpr int SPARE_OFF = NSLOT * STAGE_BYTES; // 16 KiB behind the ring: staging of a parked level, 2 KiB per wave
constexpr int NREG = TM * TN * 2;             // packed bf16x2 registers per lane per level: 32
constexpr int MAXLB = 16;
enum Kind { K_NONE = 0, K_ADD = 1, K_P0 = 2, K_P1 = 3, K_P2 = 4 };
}  // namespace wide

size_t wide_workspace_bytes(int M, int N, int lb, int split, int levels_in_registers) {
  using namespace wide;
  if (lb <= levels_in_registers) return 0;
  const size_t tiles = (size_t)((M + BM - 1) / BM) * ((N + BN - 1) / BN) * (size_t)split;
  return (size_t)(lb - levels_in_registers) * tiles * (NT / 64) * 8 * 64 * sizeof(u32x4);
}

// F16: the operands and the tree nodes are fp16 instead of bf16 (same tile, ring and order; a node is one packed add).
template <int LS, bool F16 = false, bool PAIR = false>
__global__ __launch_bounds__(wide::NT) void gemm_tree_wide_kernel(const typename WideKernelArgs<PAIR>::type pp) {
  using namespace wide;
  using NUM = Num16<F16>;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2;  // 0..1
  const int wn = wave & 3;   // 0..3

  // one problem per launch, or two (WidePair): the block index decides which one this work-group belongs to
  WideArgs p;
  int wg = blockIdx.x, nwg = gridDim.x, shard = blockIdx.y, nshards = gridDim.y;
  if constexpr (PAIR) {
    const int tiles_first = ((pp.first.M + BM - 1) / BM) * ((pp.first.N + BN - 1) / BN);
    const int wg_second = tiles_first * pp.split_first;
    const bool second = (int)blockIdx.x >= wg_second;  // wave-uniform
    p = second ? pp.second : pp.first;
    nshards = second ? pp.split_second : pp.split_first;
    nwg = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    wg = second ? blockIdx.x - wg_second : blockIdx.x;
    shard = wg / nwg;
    wg -= shard * nwg;
  } else {
    p = pp;
  }
  const int tiles_m = (p.M + BM - 1) / BM;
  const int tiles_n = (p.N + BN - 1) / BN;
  int lid = wg;
  lid = xcd_contiguous_tile(lid, nwg);
  constexpr int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int group_id = lid / per_group;
  const int first_m = group_id * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int pid_m = first_m + (lid % per_group) % gsz;
  const int pid_n = (lid % per_group) / gsz;
  const int m0 = pid_m * BM;
  const int n0 = pid_n * BN;
  const int tile_id = (shard * tiles_m + pid_m) * tiles_n + pid_n;
  const int ntiles = tiles_m * tiles_n * nshards;

  // ---- direct global->LDS loads.  Wave w's i-th load of a slice fills LDS rows [8*(8i+w), +8): lane l
  // lands at row 8*(8i+w) + l/8, physical 16-byte chunk l%8, so it fetches logical chunk (l%8)^(l/8).
  const uint8_t* xbase = reinterpret_cast<const uint8_t*>(p.X + (int64_t)m0 * p.ldx + shard * p.k_shard);
  const uint8_t* wbase = reinterpret_cast<const uint8_t*>(p.W + (int64_t)n0 * p.ldw + shard * p.k_shard);
  uint32_t voff[NDMA];
  {
    const int r = lane >> 3, c = (lane & 7) ^ r;
#pragma unroll
    for (int i = 0; i < NDMA; i++) {
      const int row = (i * 8 + wave) * 8 + r;  // 0..383
      if (i < 2) {
        const int gr = min(m0 + row, p.M - 1) - m0;
        voff[i] = (uint32_t)((gr * p.ldx + c * 8) * 2);
      } else {
        const int gr = min(n0 + row - BM, p.N - 1) - n0;
        voff[i] = (uint32_t)((gr * p.ldw + c * 8) * 2);
      }
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  auto issue_slice = [&](int s, int slot) __attribute__((always_inline)) {
    const uint8_t* xb = xbase + (int64_t)s * (BK * 2);
    const uint8_t* wb = wbase + (int64_t)s * (BK * 2);
    const uint32_t dst = lds0 + slot * STAGE_BYTES + wave * 1024;
#pragma unroll
    for (int i = 0; i < NDMA; i++) dma16(dst + i * 8192, voff[i], i < 2 ? xb : wb);
  };

  // ---- fragment addressing (bytes): lane l reads row (l%16), chunk (kk*4 + l/16) ^ (row & 7)
  const int frow = lane & 15;
  const int fchk = lane >> 4;
  const uint32_t xfrag = ((wm * TM * 16 + frow) * BK + ((fchk ^ (frow & 7)) << 3)) * 2;
  const uint32_t wfrag = (BM * BK + (wn * TN * 16 + frow) * BK + ((fchk ^ (frow & 7)) << 3)) * 2;

  f32x4 acc[TM][TN];
  uint32_t t[NREG];    // packed leaf waiting to be merged (leaf j while leaf j+1 is computed)
#pragma unroll
  for (int r = 0; r < NREG; r++) t[r] = 0;
  uint32_t s0[NREG];   // level 0 running sum
  uint32_t sb0[NREG];  // binary level 0
  int c0 = 0;          // leaves absorbed at level 0 in the current group
  int g = 0;           // groups completed
  int g_pending = 0;   // value of g for the leaf held in t

  // parked level l, 16-byte word `chunk` of this wave: a wave-uniform base (scalar registers) plus 16*lane,
  // so no per-lane pointer has to stay live across the K loop
  const uint32_t lane16 = lane * 16;
  auto ws_base = [&](int l, int chunk) __attribute__((always_inline)) -> uint8_t* {
    return reinterpret_cast<uint8_t*>(p.ws) +
           ((((int64_t)(l - RL) * ntiles + tile_id) * (NT / 64) + wave) * 8 + chunk) * (int64_t)1024;
  };
  auto ws_ptr = [&](int l, int chunk) __attribute__((always_inline)) -> u32x4* {
    return reinterpret_cast<u32x4*>(ws_base(l, chunk) + lane16);
  };

  // Parked levels for quarter q (tiles 4q..4q+3 = registers 8q..8q+7 = chunks 2q, 2q+1): continue the carry
  // chain from level `from` with counter value gg.  Stops at the first clear bit (parks there) or after lb.
  auto chain_parked = [&](int q, int from, int gg) __attribute__((always_inline)) {
    for (int l = from; l < p.lb; l++) {
      u32x4* w0 = ws_ptr(l, 2 * q);
      u32x4* w1 = ws_ptr(l, 2 * q + 1);
      if ((gg >> l) & 1) {
        const u32x4 a = *w0, b = *w1;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          t[8 * q + e] = NUM::add(a[e], t[8 * q + e]);
          t[8 * q + 4 + e] = NUM::add(b[e], t[8 * q + 4 + e]);
        }
      } else {
        store16_sbase(ws_base(l, 2 * q), lane16, u32x4{t[8 * q], t[8 * q + 1], t[8 * q + 2], t[8 * q + 3]});
        store16_sbase(ws_base(l, 2 * q + 1), lane16, u32x4{t[8 * q + 4], t[8 * q + 5], t[8 * q + 6], t[8 * q + 7]});
        break;
      }
    }
  };

  // Kinds of merge of the pending leaf (fixed per leaf, so each leaf body is straight-line code):
  //   K_ADD  s0 += t                       (group not complete)
  //   K_P0   sb0 = s0 + t                  (group complete, counter bit 0 clear)
  //   K_P1   park level 1 <- sb0 + (s0+t)  (bit 0 set, bit 1 clear)
  //   K_P2   t = lvl1 + (sb0 + (s0+t)), then the carry continues through the parked levels
  // Level 1 of quarter q arrives in the LDS staging area (prefetch_parked) before it is needed.
  const uint32_t spare_lds = lds0 + SPARE_OFF + wave * 2048;
  auto prefetch_parked = [&](int q) __attribute__((always_inline)) {
    const u32x4* src = p.ws + (((int64_t)tile_id * (NT / 64) + wave) * 8 + 2 * q) * 64;  // level RL, chunks 2q, 2q+1
    dma16(spare_lds, lane * 16, src);
    dma16(spare_lds + 1024, lane * 16, src + 64);
  };
  auto merge_quarter = [&](auto kind_c, int q) __attribute__((always_inline)) {
    constexpr int KIND = decltype(kind_c)::value;
    if (KIND == K_NONE) {
#pragma unroll
      for (int e = 0; e < 8; e++) s0[8 * q + e] = t[8 * q + e];
      return;
    }
    u32x4 pf[2];
    if (KIND == K_P2 && LS != 4) {
      pf[0] = *ws_ptr(RL, 2 * q);
      pf[1] = *ws_ptr(RL, 2 * q + 1);
    }
    if (KIND == K_P2 && LS == 4) {
      // everything older than the operand loads of this slice has landed, the staged level included
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
      pf[0] = *reinterpret_cast<const u32x4*>(smem + SPARE_OFF + wave * 2048 + lane * 16);
      pf[1] = *reinterpret_cast<const u32x4*>(smem + SPARE_OFF + wave * 2048 + 1024 + lane * 16);
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int r = 8 * q + e;
      const uint32_t l0 = NUM::add(s0[r], t[r]);
      if (KIND == K_ADD) s0[r] = l0;
      if (KIND == K_P0) sb0[r] = l0;
      if (KIND == K_P1) t[r] = NUM::add(sb0[r], l0);
      if (KIND == K_P2) t[r] = NUM::add(pf[e >> 2][e & 3], NUM::add(sb0[r], l0));
    }
    if (KIND == K_P1) {
      store16_sbase(ws_base(RL, 2 * q), lane16, u32x4{t[8 * q], t[8 * q + 1], t[8 * q + 2], t[8 * q + 3]});
      store16_sbase(ws_base(RL, 2 * q + 1), lane16, u32x4{t[8 * q + 4], t[8 * q + 5], t[8 * q + 6], t[8 * q + 7]});
    }
    if (KIND == K_P2) chain_parked(q, RL + 1, g_pending);
  };

  const int nstages = p.T * LS;
  int slot = 0;  // ring slot of the slice being consumed

  issue_slice(0, 0);
  issue_slice(min(1, nstages - 1), 1);

  // rows of the pending buffer that are merged before the last slice of a leaf (quarter q = MFMA row q)
  constexpr int EARLY_ROWS = (LS - 1) * (4 / LS);
  auto pack_row = [&](int a) __attribute__((always_inline)) {
#pragma unroll
    for (int b = 0; b < TN; b++) {
      t[(a * TN + b) * 2] = NUM::pack(acc[a][b][0], acc[a][b][1]);
      t[(a * TN + b) * 2 + 1] = NUM::pack(acc[a][b][2], acc[a][b][3]);
    }
  };
  // One leaf: LS slices of MFMAs, with the pending leaf merged a quarter (LS=4) or a half (LS=2) per slice.
  auto leaf_body = [&](auto kind_c, int j) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < LS; i++) {
      const int s = j * LS + i;
      // slice s has landed (this wave's share), then everyone's
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (decltype(kind_c)::value == K_P2 && LS == 4) prefetch_parked(i);
      // operand prefetch two slices ahead, spread over the slice: one load per four MFMAs (a burst of loads
      // right after the barrier backs up the texture path and stalls every wave behind it)
      int ns = slot + 2;
      ns = ns >= NSLOT ? ns - NSLOT : ns;
      const int ps = min(s + 2, nstages - 1);
      const uint8_t* pxb = xbase + (int64_t)ps * (BK * 2);
      const uint8_t* pwb = wbase + (int64_t)ps * (BK * 2);
      const uint32_t pdst = lds0 + ns * STAGE_BYTES + wave * 1024;
      const uint8_t* base = smem + slot * STAGE_BYTES;
#pragma unroll
      for (int kk = 0; kk < 2; kk++) {
        bf16x8 fx[TM], fw[TN];
#pragma unroll
        for (int a = 0; a < TM; a++) fx[a] = *reinterpret_cast<const bf16x8*>(base + (xfrag ^ (kk * 64)) + a * 16 * BK * 2);
#pragma unroll
        for (int b = 0; b < TN; b++) fw[b] = *reinterpret_cast<const bf16x8*>(base + (wfrag ^ (kk * 64)) + b * 16 * BK * 2);
#pragma unroll
        for (int a = 0; a < TM; a++) {
#pragma unroll
          for (int bb = 0; bb < TN; bb++) {
            // rows of tiles in alternating directions: every MFMA changes ONE of its operands
            const int b = (a & 1) ? TN - 1 - bb : bb;
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            acc[a][b] = NUM::mfma(fw[b], fx[a], (i == 0 && kk == 0) ? zero : acc[a][b]);
          }
          // The finished leaf is rounded to bf16 (into the pending buffer) one MFMA row behind the row that
          // completes it, so the rounding never waits for the MFMA pipeline; rows whose pending registers are
          // merged only at the end of this slice follow after that merge.
          if (i == LS - 1 && kk == 1 && a >= 1 && a - 1 < EARLY_ROWS) pack_row(a - 1);
          const int d = kk * TM + a;  // 0..7: loads 0..5 go out after MFMA rows 0..5
          if (d < NDMA) {
            __builtin_amdgcn_sched_barrier(0);
            dma16_at(pdst, d * 8192, voff[d], d < 2 ? pxb : pwb);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
#pragma unroll
      for (int q = i * (4 / LS); q < (i + 1) * (4 / LS); q++) merge_quarter(kind_c, q);
      if (i == LS - 1) {
#pragma unroll
        for (int a = EARLY_ROWS; a < TM; a++) pack_row(a);
      }
      slot = slot + 1 == NSLOT ? 0 : slot + 1;
    }
  };

  int kind = K_NONE;
  for (int j = 0; j < p.T; j++) {
    switch (kind) {
      case K_NONE: leaf_body(std::integral_constant<int, K_NONE>{}, j); break;
      case K_ADD: leaf_body(std::integral_constant<int, K_ADD>{}, j); break;
      case K_P0: leaf_body(std::integral_constant<int, K_P0>{}, j); break;
      case K_P1: leaf_body(std::integral_constant<int, K_P1>{}, j); break;
      default: leaf_body(std::integral_constant<int, K_P2>{}, j); break;
    }
    if (j == p.T - 1) break;  // the last leaf is packed and merged below
    // the finished leaf sits in the pending buffer; decide how it merges
    if (c0 == 0 && p.flb > 1) {
      kind = K_NONE;  // first leaf of a group: it simply becomes the running sum
      c0 = 1;
    } else if (c0 + 1 < p.flb) {
      kind = K_ADD;
      c0++;
    } else {
      // the group completes: carry through the binary counter (this is never the last group here)
      const int pops = __builtin_ctz(~g);
      kind = pops == 0 ? K_P0 : (pops == 1 ? K_P1 : K_P2);
      g_pending = g;
      g++;
      c0 = 0;
    }
  }

  // ---- the last leaf: every level carries, t ends as the root
  if (c0 != 0) {
#pragma unroll
    for (int r = 0; r < NREG; r++) t[r] = NUM::add(s0[r], t[r]);
  }
  if (p.lb > 0) {
#pragma unroll
    for (int r = 0; r < NREG; r++) t[r] = NUM::add(sb0[r], t[r]);
  }
  if (p.lb > RL) {
#pragma unroll
    for (int q = 0; q < 4; q++) chain_parked(q, RL, g);
  }

  // ---- store
#pragma unroll
  for (int a = 0; a < TM; a++) {
    const int m = m0 + (wm * TM + a) * 16 + frow;
#pragma unroll
    for (int b = 0; b < TN; b++) {
      const int n = n0 + (wn * TN + b) * 16 + fchk * 4;
      if (m >= p.M || n >= p.N) continue;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) {
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < p.N) bv[e] = NUM::to_f32(p.bias[n + e]);
      }
      uint32_t lo = t[(a * TN + b) * 2], hi = t[(a * TN + b) * 2 + 1];
      if (p.bias) {
        lo = NUM::add(lo, NUM::pack(bv[0], bv[1]));
        hi = NUM::add(hi, NUM::pack(bv[2], bv[3]));
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

static int wide_check(const WideArgs& a, int64_t* tiles) {
  using namespace wide;
  *tiles = (int64_t)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  if (*tiles <= 0 || *tiles > 0x7fffffff || a.lb > MAXLB) return TBIK_ERR_UNSUPPORTED;
  if (a.ldx >= (1 << 22) || a.ldw >= (1 << 22)) return TBIK_ERR_UNSUPPORTED;  // 32-bit in-tile byte offsets
  return TBIK_OK;
}

template <int LS, bool F16, bool PAIR>
static int wide_launch(const typename WideKernelArgs<PAIR>::type& a, dim3 grid, hipStream_t stream) {
  using namespace wide;
  constexpr size_t smem = (size_t)NSLOT * STAGE_BYTES + 16384;  // 144 KiB ring + 16 KiB staging
  auto kern = gemm_tree_wide_kernel<LS, F16, PAIR>;
  static std::atomic<uint64_t> done{0};
  hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (int)smem, done);
  if (e != hipSuccess) return hip_code(e);
  hipLaunchKernelGGL(kern, grid, dim3(NT), smem, stream, a);
  return hip_code(hipGetLastError());
}

int gemm_tree_wide_launch(const WideArgs& a, int leaf_k, bool f16, int split, hipStream_t stream) {
  int64_t tiles;
  if (const int rc = wide_check(a, &tiles)) return rc;
  const dim3 grid((unsigned)tiles, (unsigned)split);
  if (leaf_k == 256) return f16 ? wide_launch<4, true, false>(a, grid, stream) : wide_launch<4, false, false>(a, grid, stream);
  if (leaf_k == 128) return f16 ? wide_launch<2, true, false>(a, grid, stream) : wide_launch<2, false, false>(a, grid, stream);
  return TBIK_ERR_UNSUPPORTED;
}

int gemm_tree_wide_pair_launch(const WidePair& a, int leaf_k, bool f16, hipStream_t stream) {
  int64_t t1, t2;
  if (const int rc = wide_check(a.first, &t1)) return rc;
  if (const int rc = wide_check(a.second, &t2)) return rc;
  const int64_t wgs = t1 * a.split_first + t2 * a.split_second;
  if (a.split_first <= 0 || a.split_second <= 0 || wgs > 0x7fffffff) return TBIK_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)wgs);
  if (leaf_k == 256) return f16 ? wide_launch<4, true, true>(a, grid, stream) : wide_launch<4, false, true>(a, grid, stream);
  if (leaf_k == 128) return f16 ? wide_launch<2, true, true>(a, grid, stream) : wide_launch<2, false, true>(a, grid, stream);
  return TBIK_ERR_UNSUPPORTED;
}

}  // namespace tbik
