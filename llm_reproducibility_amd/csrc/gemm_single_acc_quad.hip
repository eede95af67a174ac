// Batch-invariant bf16 GEMM (one fp32 accumulator per element, K strictly ascending) for gfx950, large-M path:
// 128x256 output tile per work-group, 4 wavefronts (one per SIMD) of 64x128 each, K streamed through a 3-slot
// LDS ring in 64-element slices.  Replaces matmul_kernel_persistent, src/bio/batch_invariant_ops.py:42-124, for
// shapes that fill the chip; per element it issues the same MFMA chain as the small-tile kernel in gemm_tiled.hip,
// so the two produce identical bits and a row never sees M.
//
// Schedule (each choice measured on MI355X):
//   * one wave per SIMD with a 64x128 tile keeps the LDS traffic at 24 B per MFMA clock, below the ~31 B/clk a
//     single wave can pull from LDS (64x64 tiles need 32);
//   * operands go global -> LDS directly (global_load_lds_dwordx4), ONE load per group of four MFMAs -- bursts of
//     loads back up the texture path and stall the in-order wave -- two to three slices ahead; a lane fetches the
//     global chunk that belongs at its linear LDS position, which realises the XOR bank swizzle on the source side;
//   * one barrier per slice, placed BETWEEN its two 32-wide k steps, so fragment reads always run one k step
//     ahead of the MFMAs, also across the barrier; scheduling fences keep that order in the generated code.
#include "common.h"
#include "gemm_args.h"
#include "lds_direct.h"

namespace tbik {

namespace quad {
constexpr int BM = 128, BK = 64, NT = 256, NWAVE = 4, TM = 4;
constexpr int XDMA = BM / 8 / NWAVE;    // direct loads of X rows per wave per slice: 4 (8 rows of 128 B each)
template <int TN>
struct Shape {
  static constexpr int BN = 2 * TN * 16;          // two waves across N, TN MFMA tiles each
  static constexpr int ROWS = BM + BN;
  static constexpr int STAGE_BYTES = ROWS * BK * 2;
  static constexpr int NDMA = ROWS / 8 / NWAVE;   // direct loads per wave per slice: 12 for the 256-wide tile
};
}  // namespace quad

// TN = 8: the 128x256 tile of the large shapes.  TN = 1..4 and 6: the same pipeline on 128x32 .. 128x192 tiles for
// grids that the wide tile would not spread over the chip: the width is chosen per call so that the CUs get the same
// number of work-groups (gemm_single_acc_balanced_launch).
// NSLOT: slices of the ring.  Three keep a work-group fed when the chip is full of them; a grid of at most one narrow
// tile per CU (a handful of rows times a moderate N) is a chain of slices, each waiting for loads issued NSLOT - 1
// slices earlier, so those grids get a ring as deep as the LDS allows (5 or 6 slices).
// p.row_step < 128: a tile owns only its first row_step rows (it still stages and multiplies 128, the rest clamped to its
// last row and never stored).  For a grid that would leave most CUs without a tile: a work-group's time is its chain of
// slices whatever the rows in its tile, so the same rows spread over two to eight times the work-groups finish sooner.
template <int TN, int NSLOT>
__global__ __launch_bounds__(quad::NT) void gemm_single_acc_quad_kernel(const QuadArgs p) {
  using namespace quad;
  static_assert(NSLOT >= 3, "the schedule needs a slice in use, one landing and one in flight");
  constexpr int BN = Shape<TN>::BN, STAGE_BYTES = Shape<TN>::STAGE_BYTES, NDMA = Shape<TN>::NDMA;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  const int row_step = p.row_step > 0 ? p.row_step : BM;
  const int tiles_m = (p.M + row_step - 1) / row_step;
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
  const int m0 = pid_m * row_step, n0 = pid_n * BN;
  const int m_end = min(p.M, m0 + row_step);

  const uint8_t* xbase = reinterpret_cast<const uint8_t*>(p.X + (int64_t)m0 * p.ldx);
  const uint8_t* wbase = reinterpret_cast<const uint8_t*>(p.W + (int64_t)n0 * p.ldw);
  uint32_t voff[NDMA];
  {
    const int r = lane >> 3, c = (lane & 7) ^ r;
#pragma unroll
    for (int i = 0; i < NDMA; i++) {
      const int row = (i * NWAVE + wave) * 8 + r;  // 0..383: X rows, then W rows; rows past the edge are clamped
      if (i < XDMA) voff[i] = (uint32_t)(((min(m0 + row, m_end - 1) - m0) * p.ldx + c * 8) * 2);
      else voff[i] = (uint32_t)(((min(n0 + row - BM, p.N - 1) - n0) * p.ldw + c * 8) * 2);
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int nstages = p.K / BK;
  auto dma_one = [&](int s, int slot, int i) __attribute__((always_inline)) {
    const uint8_t* b = (i < XDMA ? xbase : wbase) + (int64_t)min(s, nstages - 1) * (BK * 2);
    dma16(lds0 + slot * STAGE_BYTES + (i * NWAVE + wave) * 1024, voff[i], b);
  };
  const int frow = lane & 15, fchk = lane >> 4;
  const uint32_t xfrag = ((wm * TM * 16 + frow) * BK + ((fchk ^ (frow & 7)) << 3)) * 2;
  const uint32_t wfrag = (BM * BK + (wn * TN * 16 + frow) * BK + ((fchk ^ (frow & 7)) << 3)) * 2;

  f32x4 acc[TM][TN];
  bf16x8 fx[2][TM], fw[2][TN];
  auto read_x = [&](int buf, int slot, int kk, int a) __attribute__((always_inline)) {
    fx[buf][a] = *reinterpret_cast<const bf16x8*>(smem + slot * STAGE_BYTES + (xfrag ^ (kk * 64)) + a * 16 * BK * 2);
  };
  auto read_w = [&](int buf, int slot, int kk, int b) __attribute__((always_inline)) {
    fw[buf][b] = *reinterpret_cast<const bf16x8*>(smem + slot * STAGE_BYTES + (wfrag ^ (kk * 64)) + b * 16 * BK * 2);
  };

  // prologue: three slices in flight, slice 0 visible, fragments of the first k step loaded
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
  for (int s = 0; s < nstages; s++) {
    const int nslot = slot + 1 == NSLOT ? 0 : slot + 1;
    const int pslot = slot == 0 ? NSLOT - 1 : slot - 1;
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      // The MFMAs of a k step go out in groups; behind every group follow two fragment reads of the next k step
      // ((s,1) from this slot, or (s+1,0) from the next slot, which the mid-slice barrier has made visible) and one
      // direct load: slice s+3 goes into the slot slice s vacates at the mid-slice barrier (first half of its loads
      // in the second k step of s, second half in the first k step of s+1).  Tiles wider than 128 columns have eight
      // groups of half a row of MFMAs each, the narrow tiles four groups of one row.
      constexpr int NG = TN > 4 ? 8 : 4;
      constexpr int H1 = (NDMA + 1) / 2, H2 = NDMA - H1;
      static_assert(H1 <= NG && TM + TN <= 2 * NG, "schedule does not fit the groups");
#pragma unroll
      for (int q = 0; q < NG; q++) {
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        const int rslot = kk == 0 ? slot : nslot;
        // the group's other instructions, each alone behind one MFMA where the group has enough of them (a wave
        // issues in order: a cluster of LDS reads and a load behind the group leaves the MFMA pipe idle meanwhile)
        auto other = [&](int j) __attribute__((always_inline)) {
          if (j < 2) {
            const int f = 2 * q + j;
            if (f < TM) read_x(kk ^ 1, rslot, kk ^ 1, f);
            else if (f - TM < TN) read_w(kk ^ 1, rslot, kk ^ 1, f - TM);
          } else {
            if (kk == 1 && q < H1) dma_one(s + NSLOT, slot, q);
            if (kk == 0 && q < H2 && s > 0) dma_one(s + NSLOT - 1, pslot, H1 + q);
          }
          __builtin_amdgcn_sched_barrier(0);
        };
        constexpr int GM = TN > 4 ? TN / 2 : TN;  // MFMAs of a group
        static_assert(TN <= 4 || TN % 2 == 0, "tiles wider than 128 columns are issued in half rows");
#pragma unroll
        for (int j = 0; j < GM; j++) {
          const int a = TN > 4 ? q >> 1 : q, b = TN > 4 ? (q & 1) * (TN / 2) + j : j;
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[kk][b], fx[kk][a], (s == 0 && kk == 0) ? zero : acc[a][b], 0, 0, 0);
          if (j < 3) other(j);
        }
#pragma unroll
        for (int j = GM; j < 3; j++) other(j);
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

#pragma unroll
  for (int a = 0; a < TM; a++) {
    const int m = m0 + (wm * TM + a) * 16 + frow;
#pragma unroll
    for (int b = 0; b < TN; b++) {
      const int n = n0 + (wn * TN + b) * 16 + fchk * 4;
      if (m >= m_end || n >= p.N) continue;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) {
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < p.N) bv[e] = bf16_bits_to_f32(p.bias[n + e]);
      }
      const uint32_t lo = pack_bf16x2(acc[a][b][0] + bv[0], acc[a][b][1] + bv[1]);
      const uint32_t hi = pack_bf16x2(acc[a][b][2] + bv[2], acc[a][b][3] + bv[3]);
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

template <int TN, int NSLOT = 3>
static int quad_launch(const QuadArgs& a, hipStream_t stream) {
  using namespace quad;
  constexpr int BN = Shape<TN>::BN;
  constexpr size_t smem = (size_t)NSLOT * Shape<TN>::STAGE_BYTES;  // 144 KiB for the 256-wide tile
  static_assert(smem <= 160 * 1024 && (NSLOT - 1) * Shape<TN>::NDMA < 64, "ring does not fit the LDS or the wait counter");
  const int row_step = a.row_step > 0 ? a.row_step : BM;
  if (row_step > BM || (row_step & 15)) return TBIK_ERR_INVALID;
  const int64_t tiles = (int64_t)((a.M + row_step - 1) / row_step) * ((a.N + BN - 1) / BN);
  if (tiles <= 0 || tiles > 0x7fffffff || a.K < BK || (a.K % BK) != 0) return TBIK_ERR_UNSUPPORTED;
  if (a.ldx >= (1 << 22) || a.ldw >= (1 << 22)) return TBIK_ERR_UNSUPPORTED;  // 32-bit in-tile byte offsets
  static std::atomic<uint64_t> done{0};
  hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_single_acc_quad_kernel<TN, NSLOT>), (int)smem, done);
  if (e != hipSuccess) return hip_code(e);
  hipLaunchKernelGGL((gemm_single_acc_quad_kernel<TN, NSLOT>), dim3((unsigned)tiles), dim3(NT), smem, stream, a);
  return hip_code(hipGetLastError());
}

int gemm_single_acc_quad_launch(const QuadArgs& a, hipStream_t stream) { return quad_launch<8>(a, stream); }

// Rows per tile for a grid of one row of tiles that leaves CUs idle: the smallest step, down to 32 rows, that still fits
// the grid into one work-group per CU (see the kernel); 0 = no split.  Measured on MI355X (cold weights, launches back to
// back): [128,4096] x [4096,4096] 22.6 -> 17.8 us, [128,8192] x [8192,2048] 38.1 -> 29.6, [96,12288] x [12288,3072]
// 60.2 -> 44.1, [64,12288] x [12288,2048] 47.3 -> 42.3.  Below 64 rows the second tile re-reads the weights for a
// handful of rows and the split loses (33 rows: 30.3 -> 32.9), and steps of 16 are no better than 32.
static int quad_row_step(int M, int64_t tiles_n) {
  if (M < 64) return 0;
  int best = 0;
  for (int step = quad::BM / 2; step >= 32; step /= 2) {
    const int64_t tm = ((int64_t)M + step - 1) / step;
    if (tm >= 2 && tiles_n * tm <= 256) best = step;
  }
  return best;
}

// 33..128 rows: one row of tiles, so the call is one pass over the weights.  A work-group's time is set by the
// length of K (the ring is a chain of slices, each about a memory round trip), not by the width of its tile, so the
// whole grid has to be resident at once: at most one work-group per CU for the 96- and 128-column tiles (84 and
// 96 KiB of LDS), two for the 32- and 64-column ones.  Among the widths that fit, the one that leaves the fewest
// of those slots idle wins (HBM bandwidth is shared about equally among the CUs), wider tiles preferred on ties
// because they re-read the activations less often.  Returns TBIK_ERR_UNSUPPORTED when no width qualifies (wide
// weight matrices run faster on the 256-column tile even with idle CUs: 110 against 214 us at N=51200).
int gemm_single_acc_slab_launch(const QuadArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.M > quad::BM) return TBIK_ERR_UNSUPPORTED;
  int best = 0;
  double best_score = 0.0;
  for (int tn = 4; tn >= 1; tn--) {
    const int64_t tiles = ((int64_t)a.N + 32 * tn - 1) / (32 * tn);
    const int64_t slots = tn <= 2 ? 512 : 256;
    if (tiles < 128 || tiles > slots) continue;
    const double score = (double)tiles / (double)(((tiles + 255) / 256) * 256) * (1.0 + 0.01 * tn);
    if (score > best_score) {
      best_score = score;
      best = tn;
    }
  }
  // at most one work-group per CU: the deep ring (see the kernel); qkv [M,4096]x[4096,6144] at M=40 27 -> 18 us, at
  // M=128 28 -> 24; [M,12288]x[12288,4096] at M=64 72 -> 49 (an eight-slice ring was measured too: no further gain)
  const bool deep = (((int64_t)a.N + 32 * best - 1) / (32 * (best ? best : 1))) <= 256;
  QuadArgs b = a;
  if (best) b.row_step = quad_row_step(a.M, ((int64_t)a.N + 32 * best - 1) / (32 * best));
  switch (best) {
    case 4: return deep ? quad_launch<4, 5>(b, stream) : quad_launch<4>(b, stream);
    case 3: return deep ? quad_launch<3, 5>(b, stream) : quad_launch<3>(b, stream);
    case 2: return deep ? quad_launch<2, 6>(b, stream) : quad_launch<2>(b, stream);
    case 1: return deep ? quad_launch<1, 6>(b, stream) : quad_launch<1>(b, stream);
    default: return TBIK_ERR_UNSUPPORTED;
  }
}

// More than 128 rows on a grid that 128x256 tiles would not spread over the chip: the tile width is chosen by a small
// cost model (constants measured on MI355X).  The mm cannot cut K (one accumulator), so a work-group's time is a pass
// over K at a per-slice rate that grows with the tile width, 0.185 + 0.0665 us per 32 columns, and by up to 16 % with
// the share of the CUs that are busy (the chip is power-bound); narrow tiles fit two work-groups on a CU, which then
// both run at 1.7 times the single rate; rounds after the first overlap the one before by about a tenth; and no
// schedule beats one pass over the weights at 3.5 TB/s.  Every width issues the same MFMA chain per element, so the
// choice never changes a bit.  Examples (us, before -> after, vendor library GEMM in brackets): qkv [M,4096]x[4096,6144]
// at M=256 39 -> 24 (37), M=512 54 -> 31 (34); gate_up (N=24576) M=384 101 -> 85 (70); 8192x8192 at M=256 83 -> 42 (68).
int gemm_single_acc_balanced_launch(const QuadArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0 || a.K < quad::BK || (a.K % quad::BK) != 0) return TBIK_ERR_UNSUPPORTED;
  const double nsl = (double)(a.K / quad::BK);
  const int64_t tm = ((int64_t)a.M + quad::BM - 1) / quad::BM;
  const double floor_us = (double)a.N * a.K * 2.0 / 3.5e6;
  static const int widths[6] = {8, 6, 4, 3, 2, 1};
  int best = 8;
  double best_t = 0.0, best_sustained = 0.0;  // the second without the overlap of later rounds (see below)
  for (int i = 0; i < 6; i++) {
    const int tn = widths[i];
    const int64_t tiles = tm * (((int64_t)a.N + 32 * tn - 1) / (32 * tn));
    const double s0 = 0.185 + 0.0665 * tn;
    double t, ts;
    if (tn <= 2) {  // up to two work-groups per CU
      if (tiles <= 256) {
        t = ts = 3.0 + nsl * s0 * (1.0 + 0.16 * (double)tiles / 256.0);
      } else {
        const double rounds = (double)((tiles + 511) / 512);
        t = (3.0 + nsl * s0 * 1.7) * (1.0 + 0.9 * (rounds - 1.0));
        ts = (3.0 + nsl * s0 * 1.7) * rounds;
      }
    } else {
      t = ts = 0.0;
      int64_t left = tiles;
      for (int r = 0; left > 0; r++, left -= 256) {
        const double fill = (double)(left < 256 ? left : 256) / 256.0;
        const double round = 3.0 + nsl * s0 * (1.0 + 0.16 * fill);
        t += (r == 0 ? 1.0 : 0.9) * round;
        ts += round;
      }
    }
    if (t < floor_us) t = floor_us + 1e-3 * t;  // memory-bound either way: keep the order of the compute estimates
    if (ts < floor_us) ts = floor_us + 1e-3 * ts;
    if (i == 0 || t < best_t) {
      best_t = t;
      best = tn;
    }
    if (i == 0 || ts < best_sustained) best_sustained = ts;
  }
  // More than one round of 128x256 tiles: the kernel with wave tiles of 128x128 (gemm_single_acc_256.hip) halves the L2
  // traffic and cuts the LDS reads per flop.  It has tiles of 256 or 192 rows by 256 or 192 columns; a round costs 6 us
  // + 1.44 / 1.17 / 1.20 / 0.94 us per slice (256x256 / 256x192 / 192x256 / 192x192, a little less on a round that does
  // not fill the chip), against 3 us + 0.83 us per slice of the 128x256 tile; the shape that wastes the fewest CU-rounds
  // wins.  The estimate above overlaps later rounds with the one before (fitted on grids of one to two rounds); a grid
  // that runs for several rounds sustains no such overlap, so the comparison uses the sum of whole rounds, and from six
  // rounds on the measured sustained rate.  gate_up [M,4096]x[4096,24576]: M=384 84 -> 67 us (256 tiles of 192x192,
  // vendor library 73), M=2048 366 -> 301, M=8192 1402 -> 1175 (272 / 1048); qkv (N=6144) at M=1536 76 -> 67 (74), at
  // M=2048 97 -> 85 (256 tiles of 256x192: one round; 84), at M=4096 177 -> 161 (159).
  {
    const int64_t tiles8 = tm * (((int64_t)a.N + 255) / 256);
    const double rounds8 = (double)((tiles8 + 255) / 256);
    static const int shape[4][2] = {{256, 256}, {256, 192}, {192, 256}, {192, 192}};
    static const double per_slice[4] = {1.44, 1.17, 1.20, 0.94};
    int pick = 0;
    double t_sq = 0.0;
    for (int i = 0; i < 4; i++) {
      int64_t left = (((int64_t)a.M + shape[i][0] - 1) / shape[i][0]) * (((int64_t)a.N + shape[i][1] - 1) / shape[i][1]);
      double t = 0.0;
      for (; left > 0; left -= 256) {
        const double fill = (double)(left < 256 ? left : 256) / 256.0;
        t += 6.0 + nsl * per_slice[i] * (1.0 + 0.16 * fill) / 1.16;
      }
      if (t < floor_us) t = floor_us + 1e-3 * t;
      if (i == 0 || t < t_sq) {
        t_sq = t;
        pick = i;
      }
    }
    const double t128 = rounds8 >= 6.0 ? rounds8 * (3.0 + nsl * 0.83) : best_sustained;
    if (tiles8 > 256 && t_sq < t128) return gemm_single_acc_256_launch(a, shape[pick][0], shape[pick][1], stream);
  }
  // at most one narrow tile per CU: the deep ring (see the kernel); qkv at M=160 31 -> 25 us, [M,12288]x[12288,4096]
  // at M=192 73 -> 51
  const bool deep = tm * (((int64_t)a.N + 32 * best - 1) / (32 * best)) <= 256;
  if (tm == 1 && best <= 4) {
    QuadArgs b = a;
    b.row_step = quad_row_step(a.M, ((int64_t)a.N + 32 * best - 1) / (32 * best));
    switch (best) {
      case 4: return quad_launch<4, 5>(b, stream);
      case 3: return quad_launch<3, 5>(b, stream);
      case 2: return quad_launch<2, 6>(b, stream);
      default: return quad_launch<1, 6>(b, stream);
    }
  }
  switch (best) {
    case 8: return quad_launch<8>(a, stream);
    case 6: return quad_launch<6>(a, stream);
    case 4: return deep ? quad_launch<4, 5>(a, stream) : quad_launch<4>(a, stream);
    case 3: return deep ? quad_launch<3, 5>(a, stream) : quad_launch<3>(a, stream);
    case 2: return deep ? quad_launch<2, 6>(a, stream) : quad_launch<2>(a, stream);
    default: return deep ? quad_launch<1, 6>(a, stream) : quad_launch<1>(a, stream);
  }
}

}  // namespace tbik
