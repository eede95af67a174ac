// Batch-invariant bf16 GEMM (one fp32 accumulator per element, K strictly ascending) for gfx950, path of the shapes
// with many rounds of tiles: 256x256 output tile per work-group, 4 wavefronts (one per SIMD) of 128x128 each, K
// streamed in 64-element slices through a ring of ten 16 KiB blocks that fills the 160 KiB of LDS.  Replaces
// matmul_kernel_persistent, src/bio/batch_invariant_ops.py:42-124, where the 128x256 tile of
// gemm_single_acc_quad.hip would make six or more rounds; per element it issues the same MFMA chain
// (v_mfma_f32_16x16x32_bf16 over k ascending into one accumulator) as every other single-accumulator kernel of this
// library, so the bits are the same and a row never sees M.
//
// Why a second tile shape: a 128x128 wave tile needs 16 fragment reads and 8 KiB of direct loads per 64 MFMAs where
// the 64x128 tile needs 24 and 12 KiB, and a work-group has half the barriers per flop.
//
// Ring: a slice of the tile is four blocks of 128 rows x 128 B (X rows of the upper and of the lower pair of waves,
// W rows of the left and of the right pair); a row is one full cache line, so the direct loads ask the L2 for whole
// lines (a ring of 32-wide units with 64 B rows doubled the L2 requests and was 8-12 % slower).  Two slices and a
// half fit: block g of the stream sits at position g mod 10.  All four blocks of slice s are free once every wave
// has read its fragments of the second k step of s, which the one barrier per slice, between its two k steps,
// establishes; into them go the W blocks of slice s+2 (issued during the second k step of s) and the X blocks of
// slice s+3 (issued during the first k step of s+1), so every load has at least the length of one k step to land
// and half of them a slice and a half.
//
// Schedule: fragment reads run one k step ahead of the MFMAs; every non-MFMA instruction sits alone behind one MFMA
// (a wave issues in order: a cluster of LDS reads and loads behind a row of MFMAs would leave the MFMA pipe idle
// while it issues).  The 16-byte chunk c of row r sits at position c ^ (r & 7); a lane of a direct load fetches the
// global chunk that belongs at its linear LDS position, which realises that swizzle on the source side.
#include <type_traits>

#include "common.h"
#include "gemm_args.h"
#include "lds_direct.h"

namespace tbik {

namespace sq {
constexpr int BK = 64, NT = 256, NWAVE = 4;
constexpr int BLOCK_BYTES = 128 * BK * 2;                          // 16 KiB: a ring position holds up to 128 rows
constexpr int NBLOCK = 10;                                         // ring positions: 160 KiB
constexpr __device__ __forceinline__ int wrap(int pos) { return pos >= NBLOCK ? pos - NBLOCK : pos; }
}  // namespace sq

// The 64 accumulator tiles of a wave are 256 registers, the whole accumulation register file.  Left to the compiler, all
// MFMA accumulators go there and, with nothing to spare, half of them are shuttled through the other file in every trip
// of the loop (two moves per MFMA).  So the MFMAs are opaque statements that pin their accumulator: seven columns of
// tiles in accumulation registers, the eighth in ordinary vector registers.  The compiler cannot see the hazards of
// such a statement: inside the loop an accumulator is touched by nothing but its own MFMA (the next one 64 MFMAs
// later), the fragment registers are written by LDS reads that the compiler orders itself, and the epilogue waits
// before anything else reads the results (mfma_results_ready).
__device__ __forceinline__ void mfma_in_agprs(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_in_vgprs(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_results_ready() {
  // an 8-pass MFMA needs up to 18 wait states before another kind of instruction may read its result; the scheduling
  // fence keeps every later instruction behind the wait
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// TM = TN = 8: 256x256 tile.  TM, TN = 6: 192 rows / columns (wave tiles of 96 rows / columns) for grids that the square
// tile does not spread evenly: the X / W blocks then hold 96 rows at the same ring positions.
template <int TM, int TN>
__global__ __launch_bounds__(sq::NT) void gemm_single_acc_256_kernel(const QuadArgs p) {
  using namespace sq;
  constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
  constexpr int XROWS = TM * 16, WROWS = TN * 16;  // rows of an X / W block
  constexpr int BDMA = XROWS / 8 / NWAVE;          // direct loads per wave per block of X (8 rows each): 4 / 3
  constexpr int WDMA = WROWS / 8 / NWAVE;          // ... of W
  constexpr int RPR = (TM + TN + TM - 1) / TM;     // fragment reads behind a row of MFMAs: 2, or 3 for the 192x256 tile
  static_assert((TM == 6 || TM == 8) && (TN == 6 || TN == 8), "tile shape");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  const int tiles_m = (p.M + BM - 1) / BM;
  const int tiles_n = (p.N + BN - 1) / BN;
  int lid = blockIdx.x;
  {
    const int nwg = gridDim.x;
    lid = xcd_contiguous_tile(lid, nwg);
  }
  constexpr int GROUP = 4;
  const int per_group = GROUP * tiles_n;
  const int group_id = lid / per_group;
  const int first_m = group_id * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int pid_m = first_m + (lid % per_group) % gsz;
  const int pid_n = (lid % per_group) / gsz;
  const int m0 = pid_m * BM, n0 = pid_n * BN;

  const uint8_t* xbase = reinterpret_cast<const uint8_t*>(p.X + (int64_t)m0 * p.ldx);
  const uint8_t* wbase = reinterpret_cast<const uint8_t*>(p.W + (int64_t)n0 * p.ldw);
  // byte offsets of this lane's direct loads inside the tile's operands: [half][load]; rows past the edge are clamped
  uint32_t voffx[2 * BDMA], voffw[2 * WDMA];
  {
    const int r = lane >> 3, c = (lane & 7) ^ r;
#pragma unroll
    for (int i = 0; i < 2 * BDMA; i++) {
      const int row = (i / BDMA) * XROWS + ((i % BDMA) * NWAVE + wave) * 8 + r;
      voffx[i] = (uint32_t)(((min(m0 + row, p.M - 1) - m0) * p.ldx + c * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < 2 * WDMA; i++) {
      const int row = (i / WDMA) * WROWS + ((i % WDMA) * NWAVE + wave) * 8 + r;
      voffw[i] = (uint32_t)(((min(n0 + row, p.N - 1) - n0) * p.ldw + c * 8) * 2);
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int nslices = p.K / BK;
  // load i (half i / BDMA, rows of load i % BDMA; WDMA for W) of the X or W blocks of slice s into ring position pos of
  // that half;
  // slices past the end of K load the last one again (never read): the count of loads in flight stays the same
  const uint32_t lds_wave = lds0 + wave * 1024;  // this wave's 1 KiB of every group of eight rows
  auto dma_x = [&](int s, int pos, int i) __attribute__((always_inline)) {
    dma16_at(lds_wave, pos * BLOCK_BYTES + (i % BDMA) * NWAVE * 1024, voffx[i], xbase + (int64_t)min(s, nslices - 1) * (BK * 2));
  };
  auto dma_w = [&](int s, int pos, int i) __attribute__((always_inline)) {
    dma16_at(lds_wave, pos * BLOCK_BYTES + (i % WDMA) * NWAVE * 1024, voffw[i], wbase + (int64_t)min(s, nslices - 1) * (BK * 2));
  };
  const int frow = lane & 15, fchk = lane >> 4;
  const uint32_t frag = (frow * BK + ((fchk ^ (frow & 7)) << 3)) * 2;  // inside a block, row a * 16 + frow, k step 0

  f32x4 acc[TM][TN];
  bf16x8 fx[2][TM], fw[2][TN];
  // this wave's fragment addresses inside the first X block / W block of a slice (its half selects the block)
  const uint32_t xfrag = frag + wm * BLOCK_BYTES, wfrag = frag + wn * BLOCK_BYTES;
  // fragment f (X rows first) of k step kk of the slice whose first block sits at ring position px (a constant)
  auto read_frag = [&](int buf, int px, int kk, int f) __attribute__((always_inline)) {
    if (f < TM) fx[buf][f] = *reinterpret_cast<const bf16x8*>(smem + (xfrag ^ (kk * 64)) + px * BLOCK_BYTES + f * 16 * BK * 2);
    else fw[buf][f - TM] = *reinterpret_cast<const bf16x8*>(smem + (wfrag ^ (kk * 64)) + wrap(px + 2) * BLOCK_BYTES + (f - TM) * 16 * BK * 2);
  };

  // prologue: slices 0 and 1 and the X blocks of slice 2 fill the ten positions; slice 0 visible, fragments of its
  // first k step in registers
#pragma unroll
  for (int s = 0; s < 2; s++) {
#pragma unroll
    for (int i = 0; i < 2 * BDMA; i++) dma_x(s, 4 * s + i / BDMA, i);
#pragma unroll
    for (int i = 0; i < 2 * WDMA; i++) dma_w(s, 4 * s + 2 + i / WDMA, i);
  }
#pragma unroll
  for (int i = 0; i < 2 * BDMA; i++) dma_x(2, 8 + i / BDMA, i);
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++) {
      // zero here, long before the first MFMA, and opaque from here on: a zero that the compiler knows to be zero is
      // written again right in front of the first MFMA, closer than an MFMA may follow a write of its accumulator
      acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (TN < 8 || b < TN - 1) asm volatile("" : "+a"(acc[a][b]));
      else asm volatile("" : "+v"(acc[a][b]));
    }
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(4 * BDMA + 2 * WDMA) : "memory");  // all but slice 0
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int f = 0; f < TM + TN; f++) read_frag(0, 0, 0, f);

  // One slice; PX, the ring position of its first block, is a constant: the positions repeat every five slices, so the
  // loop below takes five slices per trip and no instruction is spent on ring arithmetic.
  auto slice = [&](auto px_c, int s) __attribute__((always_inline)) {
    constexpr int px = decltype(px_c)::value, px1 = wrap(px + 4);
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
#pragma unroll
      for (int q = 0; q < TM; q++) {
#pragma unroll
        for (int b = 0; b < TN; b++) {
          if (TN < 8 || b < TN - 1) mfma_in_agprs(acc[q][b], fw[kk][b], fx[kk][q]);
          else mfma_in_vgprs(acc[q][b], fw[kk][b], fx[kk][q]);
          if (b < 2 * RPR - 1 && (RPR == 3 || (b & 1) == 0)) {
            // fragments of the next k step: the second of this slice, or the first of the next slice (behind the
            // last slice that reads blocks whose loads have landed and are never used)
            const int f = RPR * q + (RPR == 3 ? b : b >> 1);
            if (f < TM + TN) {
              if (kk == 0) read_frag(1, px, 1, f);
              else read_frag(0, px1, 0, f);
            }
          }
          if (b == 4 || b == 6) {
            // first k step: X blocks of slice s+2 into the positions of the W blocks of slice s-1 (the prologue has
            // issued those of slice 2); second k step: W blocks of slice s+2 into the positions of the X blocks of s.
            // One load behind the fifth MFMA of every row, and where a k step has more loads than rows (the 192x256
            // tile) the rest behind the seventh MFMA of the first rows
            const int d = b == 4 ? q : TM + q;
            if (kk == 0) {
              if (s > 0 && d < 2 * BDMA) dma_x(s + 2, wrap(px + 8) + d / BDMA, d);
            } else if (d < 2 * WDMA) {
              dma_w(s + 2, px + d / WDMA, d);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (kk == 0) {
        // between the k steps: slice s+1 has landed (this wave's share: the X loads of s+2 may still fly) and every
        // fragment read of slice s is done
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * BDMA) : "memory");
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
      }
    }
  };
  for (int s = 0; s < nslices; s += 5) {
    slice(std::integral_constant<int, 0>{}, s);
    if (s + 1 >= nslices) break;
    slice(std::integral_constant<int, 4>{}, s + 1);
    if (s + 2 >= nslices) break;
    slice(std::integral_constant<int, 8>{}, s + 2);
    if (s + 3 >= nslices) break;
    slice(std::integral_constant<int, 2>{}, s + 3);
    if (s + 4 >= nslices) break;
    slice(std::integral_constant<int, 6>{}, s + 4);
  }

  mfma_results_ready();
  // Tiles that lie inside N and whose rows allow 16-byte stores go through the LDS (the ring is done with): a lane of
  // an MFMA tile owns four columns of one row, 8 bytes, and sixteen rows at a time make a store of sixteen 32-byte
  // pieces; read back row by row, sixteen lanes store one 256-byte row of the wave's tile, whole cache lines.  All
  // work-groups of a round finish together, so their stores are one burst that the next round's loads queue behind.
  const bool rows_by_16_bytes = n0 + BN <= p.N && (p.ldc & 7) == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
  if (rows_by_16_bytes) {
    constexpr int ROWB = TN * 32 + 16;  // bytes per row of a wave's tile, padded against bank conflicts
    static_assert(NWAVE * TM * 16 * ROWB <= NBLOCK * BLOCK_BYTES, "staging does not fit");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the loads past the end of K still write into the ring
    __builtin_amdgcn_s_barrier();                    // ... and no wave reads it any more
    uint8_t* stage = smem + wave * (TM * 16 * ROWB);
#pragma unroll
    for (int a = 0; a < TM; a++) {
#pragma unroll
      for (int b = 0; b < TN; b++) {
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.bias) {
          const int n = n0 + (wn * TN + b) * 16 + fchk * 4;
#pragma unroll
          for (int e = 0; e < 4; e++) bv[e] = bf16_bits_to_f32(p.bias[n + e]);
        }
        const uint32_t lo = pack_bf16x2(acc[a][b][0] + bv[0], acc[a][b][1] + bv[1]);
        const uint32_t hi = pack_bf16x2(acc[a][b][2] + bv[2], acc[a][b][3] + bv[3]);
        *reinterpret_cast<uint2*>(stage + (a * 16 + frow) * ROWB + (b * 16 + fchk * 4) * 2) = make_uint2(lo, hi);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // a wave reads back only what it wrote itself
    const int rl = lane / (TN * 2), cl = lane % (TN * 2);  // TN * 2 lanes of 16 bytes per row
    constexpr int RPI = 64 / (TN * 2);                   // rows per instruction: 4, or 5 of which lanes 60..63 idle
#pragma unroll
    for (int j = 0; j < (TM * 16 + RPI - 1) / RPI; j++) {
      const int row = j * RPI + rl;
      const int m = m0 + wm * TM * 16 + row;
      if (rl < RPI && row < TM * 16 && m < p.M) {
        const uint4 v = *reinterpret_cast<const uint4*>(stage + row * ROWB + cl * 16);
        *reinterpret_cast<uint4*>(p.C + (int64_t)m * p.ldc + n0 + wn * TN * 16 + cl * 8) = v;
      }
    }
    return;
  }
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
  // the direct loads past the end of K have an address in this work-group's LDS: they must land before it is released
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int TM, int TN>
static int sq_launch(const QuadArgs& a, hipStream_t stream) {
  using namespace sq;
  constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
  constexpr size_t smem = (size_t)NBLOCK * BLOCK_BYTES;  // 160 KiB: all of a CU's LDS
  const int64_t tiles = (int64_t)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  if (tiles <= 0 || tiles > 0x7fffffff || a.K < BK || (a.K % BK) != 0) return TBIK_ERR_UNSUPPORTED;
  if (a.ldx >= (1 << 22) || a.ldw >= (1 << 22)) return TBIK_ERR_UNSUPPORTED;  // 32-bit in-tile byte offsets
  static std::atomic<uint64_t> done{0};
  hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_single_acc_256_kernel<TM, TN>), (int)smem, done);
  if (e != hipSuccess) return hip_code(e);
  hipLaunchKernelGGL((gemm_single_acc_256_kernel<TM, TN>), dim3((unsigned)tiles), dim3(NT), smem, stream, a);
  return hip_code(hipGetLastError());
}

int gemm_single_acc_256_launch(const QuadArgs& a, int tile_rows, int tile_cols, hipStream_t stream) {
  if (tile_rows == 256 && tile_cols == 256) return sq_launch<8, 8>(a, stream);
  if (tile_rows == 256 && tile_cols == 192) return sq_launch<8, 6>(a, stream);
  if (tile_rows == 192 && tile_cols == 256) return sq_launch<6, 8>(a, stream);
  if (tile_rows == 192 && tile_cols == 192) return sq_launch<6, 6>(a, stream);
  return TBIK_ERR_UNSUPPORTED;
}

}  // namespace tbik
