// Tree-ordered bf16 GEMM for gfx950, large-M path for trees that carry often (leaf 256; four or more binary levels, or
// two or more when a group has two leaves): the same tile, ring and arithmetic as gemm_tree_wide.hip (128x256 output
// tile per work-group, 8 wavefronts of 64x64, K streamed through a 3-slot LDS ring in 64-element slices, one chain of
// 16x16x32 bf16 MFMAs per leaf, one rounding per leaf, every tree node rounded to bf16), so the bits are the same;
// what differs is where the merge tree lives:
//   * TWO binary levels stay in registers next to the level-0 running sum (the other kernel keeps one), so a tree of 16
//     groups parks a level in the workspace 3 times instead of 7 and meets a parked level once instead of 3 times;
//   * ONE loop body serves every leaf: what happens to the previous leaf (nothing / add to the running sum / one of
//     the carries) is decided by wave-uniform branches around the merge code of each slice, and a leaf that opens a
//     group is rounded straight into the running-sum registers.  With a single body the register allocator keeps every
//     array in place across the loop (no copies at the joins of per-kind bodies), which is what makes room for the
//     second level inside the 256 registers of a wave; the price is a few scalar branches per slice, so trees that
//     carry less often stay on the other kernel.
// Replaces matmul_kernel_tp_persistent, src/tbik/tree_based_matmul.py:50-187.
//
// This file is compiled with -structurizecfg-skip-uniform-regions: the branches in the K loop are wave-uniform, and
// leaving them unstructured keeps the compiler from turning them into chains of flow blocks with a copy per live
// register.
#include "common.h"
#include "gemm_args.h"
#include "lds_direct.h"

namespace tbik {

namespace deep {
constexpr int BM = 128, BN = 256, BK = 64;
constexpr int NT = 512;
constexpr int TM = 4, TN = 4;                 // 16x16 MFMA tiles per wave: 64x64
constexpr int ROWS = BM + BN;                 // LDS rows per slice: X rows, then W rows
constexpr int STAGE_BYTES = ROWS * BK * 2;    // 48 KiB
constexpr int NSLOT = 3;
constexpr int NDMA = ROWS / 8 / (NT / 64);    // direct loads per wave per slice: 6 (8 rows of 128 B each)
constexpr int LS = 4;                         // slices per leaf of 256
constexpr int RL = 2;                         // binary levels kept in registers
constexpr int SPARE_OFF = NSLOT * STAGE_BYTES; // 16 KiB behind the ring: staging of a parked level, 2 KiB per wave
constexpr int NREG = TM * TN * 2;             // packed bf16x2 registers per lane per level: 32
constexpr int MAXLB = 16;
enum Kind { K_NONE = 0, K_ADD = 1, K_P0 = 2, K_P1 = 3, K_P2 = 4 };
}  // namespace deep

template <bool PAIR>
__global__ __launch_bounds__(deep::NT) void gemm_tree_deep_kernel(const typename WideKernelArgs<PAIR>::type pp) {
  using namespace deep;
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
  uint32_t t[NREG];    // packed leaf waiting to be merged
  uint32_t s0[NREG];   // level 0: running sum of the current group
  uint32_t sb0[NREG];  // binary level 0
  uint32_t sb1[NREG];  // binary level 1
#pragma unroll
  for (int r = 0; r < NREG; r++) t[r] = s0[r] = sb0[r] = sb1[r] = 0;

  const uint32_t lane16 = lane * 16;
  auto ws_base = [&](int l, int chunk) __attribute__((always_inline)) -> uint8_t* {
    return reinterpret_cast<uint8_t*>(p.ws) +
           ((((int64_t)(l - RL) * ntiles + tile_id) * (NT / 64) + wave) * 8 + chunk) * (int64_t)1024;
  };
  auto ws_ptr = [&](int l, int chunk) __attribute__((always_inline)) -> u32x4* {
    return reinterpret_cast<u32x4*>(ws_base(l, chunk) + lane16);
  };
  auto chain_parked = [&](int q, int from, int gg) __attribute__((always_inline)) {
    for (int l = from; l < p.lb; l++) {
      u32x4* w0 = ws_ptr(l, 2 * q);
      u32x4* w1 = ws_ptr(l, 2 * q + 1);
      if ((gg >> l) & 1) {
        const u32x4 a = *w0, b = *w1;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          t[8 * q + e] = add_bf16x2(a[e], t[8 * q + e]);
          t[8 * q + 4 + e] = add_bf16x2(b[e], t[8 * q + 4 + e]);
        }
      } else {
        store16_sbase(ws_base(l, 2 * q), lane16, u32x4{t[8 * q], t[8 * q + 1], t[8 * q + 2], t[8 * q + 3]});
        store16_sbase(ws_base(l, 2 * q + 1), lane16, u32x4{t[8 * q + 4], t[8 * q + 5], t[8 * q + 6], t[8 * q + 7]});
        break;
      }
    }
  };
  const uint32_t spare_lds = lds0 + SPARE_OFF + wave * 2048;
  auto prefetch_parked = [&](int q) __attribute__((always_inline)) {
    const u32x4* src = p.ws + (((int64_t)tile_id * (NT / 64) + wave) * 8 + 2 * q) * 64;  // level RL, chunks 2q, 2q+1
    dma16(spare_lds, lane * 16, src);
    dma16(spare_lds + 1024, lane * 16, src + 64);
  };

  // Leaf state.  pos: position of the leaf being multiplied in its group of flb leaves; kind: what happens to the
  // leaf that was finished before it (held in t, or already in s0 when it was the first of its group):
  //   K_NONE nothing;  K_ADD s0 += t;  K_P0 sb0 = s0 + t;  K_P1 sb1 = sb0 + (s0 + t);
  //   K_P2 t = sb1 + (sb0 + (s0 + t)), which is parked at level 2 or, when a value waits there, carries on through
  //   the parked levels.
  // The first leaf of a group is rounded straight into s0 (the completion merge has consumed the old s0 by then).
  int pos = 0, kind = K_NONE, g = 0, g_pending = 0;

  // merge of quarter q (MFMA row q of the wave's tile: registers 8q..8q+7 of every level)
  auto merge_in_registers = [&](int q) __attribute__((always_inline)) {
    if (kind == K_ADD) {
#pragma unroll
      for (int e = 0; e < 8; e++) s0[8 * q + e] = add_bf16x2(s0[8 * q + e], t[8 * q + e]);
    } else if (kind == K_P0) {
#pragma unroll
      for (int e = 0; e < 8; e++) sb0[8 * q + e] = add_bf16x2(s0[8 * q + e], t[8 * q + e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) sb1[8 * q + e] = add_bf16x2(sb0[8 * q + e], add_bf16x2(s0[8 * q + e], t[8 * q + e]));
    }
  };
  auto merge_through_workspace = [&](int q) __attribute__((always_inline)) {
    // bits 0 and 1 of the group counter are set: t = sb1 + (sb0 + (s0 + t)); bit 2 decides whether that value is
    // parked at level 2 or meets the value parked there (staged in LDS since the start of this slice) and carries on
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int r = 8 * q + e;
      t[r] = add_bf16x2(sb1[r], add_bf16x2(sb0[r], add_bf16x2(s0[r], t[r])));
    }
    if ((g_pending >> RL) & 1) {
      u32x4 pf[2];
      // everything older than the operand loads of this slice has landed, the staged level included
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
      pf[0] = *reinterpret_cast<const u32x4*>(smem + SPARE_OFF + wave * 2048 + lane * 16);
      pf[1] = *reinterpret_cast<const u32x4*>(smem + SPARE_OFF + wave * 2048 + 1024 + lane * 16);
#pragma unroll
      for (int e = 0; e < 8; e++) t[8 * q + e] = add_bf16x2(pf[e >> 2][e & 3], t[8 * q + e]);
      chain_parked(q, RL + 1, g_pending);
    } else {
      store16_sbase(ws_base(RL, 2 * q), lane16, u32x4{t[8 * q], t[8 * q + 1], t[8 * q + 2], t[8 * q + 3]});
      store16_sbase(ws_base(RL, 2 * q + 1), lane16, u32x4{t[8 * q + 4], t[8 * q + 5], t[8 * q + 6], t[8 * q + 7]});
    }
  };

  // rows of the pending buffer whose merge is over before the last slice of a leaf even when it runs at slice ends
  constexpr int EARLY_ROWS = 3;
  const int nstages = p.T * LS;
  int slot = 0;

  issue_slice(0, 0);
  issue_slice(min(1, nstages - 1), 1);

  for (int j = 0; j < p.T; j++) {
    const bool to_s0 = pos == 0;
    const bool simple = kind == K_ADD || kind == K_P0 || kind == K_P1;  // merges that stay in registers
    const bool park = kind == K_P2;                                     // merges that touch the workspace
    auto pack_row = [&](int a) __attribute__((always_inline)) {
      if (to_s0) {
#pragma unroll
        for (int b = 0; b < TN; b++) {
          // the empty statements keep the two arms distinct (otherwise the conversions are hoisted in front of the
          // branch and copied into place) and the results where they are computed (otherwise they sink to the loop end)
          float c0 = acc[a][b][0], c1 = acc[a][b][1], c2 = acc[a][b][2], c3 = acc[a][b][3];
          asm volatile("" : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3));
          s0[(a * TN + b) * 2] = pack_bf16x2(c0, c1);
          s0[(a * TN + b) * 2 + 1] = pack_bf16x2(c2, c3);
          asm volatile("" : "+v"(s0[(a * TN + b) * 2]), "+v"(s0[(a * TN + b) * 2 + 1]));
        }
      } else {
#pragma unroll
        for (int b = 0; b < TN; b++) {
          t[(a * TN + b) * 2] = pack_bf16x2(acc[a][b][0], acc[a][b][1]);
          t[(a * TN + b) * 2 + 1] = pack_bf16x2(acc[a][b][2], acc[a][b][3]);
          asm volatile("" : "+v"(t[(a * TN + b) * 2]), "+v"(t[(a * TN + b) * 2 + 1]));
        }
      }
    };
#pragma unroll
    for (int i = 0; i < LS; i++) {
      const int s = j * LS + i;
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (park && ((g_pending >> RL) & 1)) prefetch_parked(i);
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
        // the register-only merge of quarter i sits between the fragment loads of the second k step and its MFMAs,
        // where it covers the latency of those loads
        if (kk == 1 && simple) {
          __builtin_amdgcn_sched_barrier(0);
          merge_in_registers(i);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int a = 0; a < TM; a++) {
#pragma unroll
          for (int bb = 0; bb < TN; bb++) {
            // rows of tiles in alternating directions: every MFMA then changes ONE of its operands, never both at the
            // turn of a row (an MFMA-only loop on random operands runs 2 % faster at the same power this way)
            const int b = (a & 1) ? TN - 1 - bb : bb;
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[b], fx[a], (i == 0 && kk == 0) ? zero : acc[a][b], 0, 0, 0);
          }
          // the finished leaf is rounded to bf16 one MFMA row behind the row that completes it
          if (i == LS - 1 && kk == 1 && a >= 1 && (a - 1 < EARLY_ROWS || !park)) pack_row(a - 1);
          const int d = kk * TM + a;
          if (d < NDMA) {
            __builtin_amdgcn_sched_barrier(0);
            dma16_at(pdst, d * 8192, voff[d], d < 2 ? pxb : pwb);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      if (park) merge_through_workspace(i);
      if (i == LS - 1) {
        if (park) {
#pragma unroll
          for (int a = EARLY_ROWS; a < TM - 1; a++) pack_row(a);
        }
        pack_row(TM - 1);
      }
      slot = slot + 1 == NSLOT ? 0 : slot + 1;
    }
    // what happens to the leaf just finished, while the next one is multiplied
    if (pos == 0 && p.flb > 1) {
      kind = K_NONE;
      pos = 1;
    } else if (pos + 1 < p.flb) {
      kind = K_ADD;
      pos++;
    } else {
      const int pops = __builtin_ctz(~g);
      kind = pops == 0 ? K_P0 : (pops == 1 ? K_P1 : K_P2);
      g_pending = g;
      g++;
      pos = 0;
    }
  }

  // ---- the last leaf completes the last group: every level carries, t ends as the root
  if (p.flb > 1) {
#pragma unroll
    for (int r = 0; r < NREG; r++) t[r] = add_bf16x2(s0[r], t[r]);
  } else {
#pragma unroll
    for (int r = 0; r < NREG; r++) t[r] = s0[r];
  }
  if (p.lb > 0) {
#pragma unroll
    for (int r = 0; r < NREG; r++) t[r] = add_bf16x2(sb0[r], t[r]);
  }
  if (p.lb > 1) {
#pragma unroll
    for (int r = 0; r < NREG; r++) t[r] = add_bf16x2(sb1[r], t[r]);
  }
  if (p.lb > RL) {
#pragma unroll
    for (int q = 0; q < 4; q++) chain_parked(q, RL, g - 1);
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
          if (n + e < p.N) bv[e] = bf16_bits_to_f32(p.bias[n + e]);
      }
      uint32_t lo = t[(a * TN + b) * 2], hi = t[(a * TN + b) * 2 + 1];
      if (p.bias) {
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

static int deep_check(const WideArgs& a, int64_t* tiles) {
  using namespace deep;
  *tiles = (int64_t)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  if (*tiles <= 0 || *tiles > 0x7fffffff || a.lb > MAXLB) return TBIK_ERR_UNSUPPORTED;
  if (a.ldx >= (1 << 22) || a.ldw >= (1 << 22)) return TBIK_ERR_UNSUPPORTED;  // 32-bit in-tile byte offsets
  return TBIK_OK;
}

int gemm_tree_deep_launch(const WideArgs& a, int split, hipStream_t stream) {
  using namespace deep;
  constexpr size_t smem = (size_t)NSLOT * STAGE_BYTES + 16384;  // 144 KiB ring + 16 KiB staging
  int64_t tiles;
  if (const int rc = deep_check(a, &tiles)) return rc;
  auto kern = gemm_tree_deep_kernel<false>;
  static std::atomic<uint64_t> done{0};
  hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (int)smem, done);
  if (e != hipSuccess) return hip_code(e);
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)split), dim3(NT), smem, stream, a);
  return hip_code(hipGetLastError());
}

int gemm_tree_deep_pair_launch(const WidePair& a, hipStream_t stream) {
  using namespace deep;
  constexpr size_t smem = (size_t)NSLOT * STAGE_BYTES + 16384;
  int64_t t1, t2;
  if (const int rc = deep_check(a.first, &t1)) return rc;
  if (const int rc = deep_check(a.second, &t2)) return rc;
  const int64_t wgs = t1 * a.split_first + t2 * a.split_second;
  if (a.split_first <= 0 || a.split_second <= 0 || wgs > 0x7fffffff) return TBIK_ERR_UNSUPPORTED;
  auto kern = gemm_tree_deep_kernel<true>;
  static std::atomic<uint64_t> done{0};
  hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (int)smem, done);
  if (e != hipSuccess) return hip_code(e);
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(NT), smem, stream, a);
  return hip_code(hipGetLastError());
}

}  // namespace tbik
