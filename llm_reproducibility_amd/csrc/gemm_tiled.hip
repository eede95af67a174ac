// Tiled bf16 MFMA GEMM for gfx950 with two accumulation disciplines:
//
//   TREE = true   tree-ordered (TP-invariant) GEMM.  K is cut into leaves of LS*64 elements; a leaf is
//                 a chain of 16x16x32 bf16 MFMAs into a zeroed fp32 accumulator, rounded once to bf16;
//                 leaves merge through a binary-counter stack of packed-bf16 partials held in registers
//                 (level 0: left-to-right over FLB leaves, levels above: adjacent pairs), every node
//                 rounded to bf16.  Replaces matmul_kernel_tp_persistent,
//                 src/tbik/tree_based_matmul.py:50-187 of the reference.
//   TREE = false  one fp32 accumulator per element run sequentially over all of K (batch-invariant mm),
//                 replaces matmul_kernel_persistent, src/bio/batch_invariant_ops.py:42-124.
//
// Invariance argument: the value of C[m,n] is produced by ONE lane's accumulator registers from the
// k-ordered MFMA chain on row m of A and row n of W; tile sizes, wave placement, padding rows and
// the block->tile map only decide WHICH lane does it.  All tile configurations therefore give the
// same bits, and row m never sees M.
//
// Operand roles: W ([N,K], K contiguous) feeds the MFMA "A" port and X ([M,K]) the "B" port, so an
// output lane holds 4 consecutive n of one m and stores them as one 8-byte word.
//
// WT = true: the weight operand is given row-major as B[K,N] (N contiguous, row stride ldw) -- what a plain
// `x @ B` hands over (simple_matmul.py:11-14 of the reference; the reference kernel takes B's strides as they are,
// src/tbik/tree_based_matmul.py:259-264).  It is consumed in place: a thread loads an 8(k) x 8(n) block as eight
// 16-byte rows, transposes it in registers (v_perm_b32) and writes eight K-contiguous 16-byte chunks into the same
// LDS tile layout, so fragments, MFMA chain and bits are those of the [N,K] form.
#include <algorithm>

#include "common.h"
#include "gemm_args.h"

namespace tbik {

struct GemmArgs {
  const uint16_t* X;   // [M,K], row stride ldx
  const uint16_t* W;   // [N,K], row stride ldw
  uint16_t* C;         // [M,N], row stride ldc
  const uint16_t* bias;
  int64_t ldx, ldw, ldc;
  int M, N, K;
  int T;      // leaves (TREE)
  int flb;    // leaves summed left to right at level 0
  int lb;     // binary levels above level 0
  int vec_store;  // C rows allow 8-byte stores
  // K split into gridDim.y shards (aligned subtrees): shard y reads columns [y*k_shard, +K) of X and W and writes
  // its bf16 partial at C + y*c_shard; the shard tree (tree_combine) then rebuilds the unsplit result bit for bit
  int64_t k_shard, c_shard;
};

constexpr int BK = 64;  // K elements per LDS stage (8 chunks of 16 bytes per row)

// Element offset of 16-byte chunk `c` (0..7) of tile row `r` in an LDS tile of 64-element rows.
// The XOR spreads the 16 rows an MFMA fragment read touches over all banks.
__device__ __forceinline__ int lds_off(int r, int c) { return r * BK + ((c ^ (r & 7)) << 3); }

template <int WAVES_M, int WAVES_N, int TM, int TN, int LS, int LBMAX, bool TREE, bool F16, bool WT = false>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_kernel(const GemmArgs p) {
  using Num = Num16<F16>;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * TM * 16;
  constexpr int BN = WAVES_N * TN * 16;
  constexpr int XCH = (BM * 8 + NT - 1) / NT;  // 16-byte chunks of the X tile per thread
  constexpr int WCH = WT ? 8 : (BN * 8 + NT - 1) / NT;  // WT: the eight k rows of this thread's 8x8 block
  static_assert(!WT || NT >= BN, "one 8x8 block of the W tile per thread");

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  constexpr int STAGE = (BM + BN) * BK;  // elements per LDS stage: X tile, then W tile

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N;
  const int wn = wave % WAVES_N;

  // ---- block -> tile: consecutive logical ids stay on one XCD (blocks are dealt round-robin over the
  // 8 XCDs), and walk the tile grid in bands of 8 m-tiles so an XCD's L2 sees few distinct panels.
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
  const int m0 = pid_m * BM;
  const int n0 = pid_n * BN;

  const uint16_t* Xs = p.X + blockIdx.y * p.k_shard;
  const uint16_t* Ws = p.W + blockIdx.y * p.k_shard * (WT ? p.ldw : 1);
  uint16_t* Cs = p.C + blockIdx.y * p.c_shard;

  // ---- global -> register staging (rows past the edge are clamped: their results are never stored)
  const uint16_t* xptr[XCH];
  const uint16_t* wptr[WCH];
  int xdst[XCH], wdst[WCH];
#pragma unroll
  for (int i = 0; i < XCH; i++) {
    const int q = tid + i * NT;
    const int r = (q >> 3) % BM, c = q & 7;
    const int gr = min(m0 + r, p.M - 1);
    xptr[i] = Xs + (int64_t)gr * p.ldx + c * 8;
    xdst[i] = lds_off(r, c);
  }
  // WT: thread b < BN owns the block of k rows 8*(b%8) .. +7 and columns 8*(b/8) .. +7 of the tile (eight lanes
  // that differ in the k block read one full 128-byte line of each of eight k rows and write one LDS row)
  const int wt_kb = tid & 7, wt_nb = tid >> 3;
  const bool wt_active = WT && tid < BN;
  const bool wt_full = WT && (n0 + wt_nb * 8 + 8 <= p.N);   // else: the block crosses the edge, loaded element-wise
#pragma unroll
  for (int i = 0; i < WCH; i++) {
    if (WT) {
      wptr[i] = Ws + (int64_t)(wt_kb * 8 + i) * p.ldw + n0 + wt_nb * 8;
      wdst[i] = lds_off(wt_nb * 8 + i, wt_kb);   // destination of the transposed chunk for column 8*nb + i
    } else {
      const int q = tid + i * NT;
      const int r = (q >> 3) % BN, c = q & 7;
      const int gr = min(n0 + r, p.N - 1);
      wptr[i] = Ws + (int64_t)gr * p.ldw + c * 8;
      wdst[i] = lds_off(r, c);
    }
  }
  // Staging registers.  Large tree tiles load one stage ahead (their merge stack needs the registers); the
  // single-accumulator mm (no K split, so often a small grid in which every work-group is a chain of memory round
  // trips) and the small tree tiles of decode-sized M load two stages ahead into two register sets that alternate
  // with the parity of the stage.
  constexpr int NSET = (TREE && TM * TN > 8) ? 1 : 2;
  u32x4 xregs[NSET][XCH], wregs[NSET][WCH];

  auto load_stage = [&](int s, int set) __attribute__((always_inline)) {
    u32x4* xreg = xregs[set];
    u32x4* wreg = wregs[set];
    const int k0 = s * BK;
#pragma unroll
    for (int i = 0; i < XCH; i++) {
      if ((BM * 8) % NT == 0 || tid + i * NT < BM * 8) {
        if (TREE || k0 + (tid & 7) * 8 < p.K)
          xreg[i] = *reinterpret_cast<const u32x4*>(xptr[i] + k0);
        else
          xreg[i] = u32x4{0, 0, 0, 0};
      }
    }
    if (WT) {
      if (wt_active) {
        const bool k_ok = TREE || k0 + wt_kb * 8 < p.K;   // K is a multiple of 8: a block is inside or outside
#pragma unroll
        for (int i = 0; i < WCH; i++) {
          const uint16_t* src = wptr[i] + (int64_t)k0 * p.ldw;
          if (!k_ok) {
            wreg[i] = u32x4{0, 0, 0, 0};
          } else if (wt_full) {
            wreg[i] = *reinterpret_cast<const u32x4*>(src);
          } else {
            uint32_t w4[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const int c0 = min(n0 + wt_nb * 8 + 2 * e, p.N - 1) - (n0 + wt_nb * 8);      // clamped: never stored
              const int c1 = min(n0 + wt_nb * 8 + 2 * e + 1, p.N - 1) - (n0 + wt_nb * 8);
              w4[e] = (uint32_t)src[c0] | ((uint32_t)src[c1] << 16);
            }
            wreg[i] = u32x4{w4[0], w4[1], w4[2], w4[3]};
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < WCH; i++) {
        if ((BN * 8) % NT == 0 || tid + i * NT < BN * 8) {
          if (TREE || k0 + (tid & 7) * 8 < p.K)
            wreg[i] = *reinterpret_cast<const u32x4*>(wptr[i] + k0);
          else
            wreg[i] = u32x4{0, 0, 0, 0};
        }
      }
    }
  };
  auto store_stage = [&](int buf, int set) __attribute__((always_inline)) {
    const u32x4* xreg = xregs[set];
    const u32x4* wreg = wregs[set];
#pragma unroll
    for (int i = 0; i < XCH; i++)
      if ((BM * 8) % NT == 0 || tid + i * NT < BM * 8) *reinterpret_cast<u32x4*>(smem + buf * STAGE + xdst[i]) = xreg[i];
    if (WT) {
      if (wt_active) {
        // 8x8 transpose of 16-bit elements: column j of the block = (row 0..7).half[j]; word w of the output pairs
        // k rows 2w and 2w+1 (low half = the even row)
#pragma unroll
        for (int j = 0; j < 8; j++) {
          u32x4 o;
#pragma unroll
          for (int w = 0; w < 4; w++)
            o[w] = __builtin_amdgcn_perm(wreg[2 * w + 1][j >> 1], wreg[2 * w][j >> 1], (j & 1) ? 0x07060302u : 0x05040100u);
          *reinterpret_cast<u32x4*>(smem + buf * STAGE + BM * BK + wdst[j]) = o;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < WCH; i++)
        if ((BN * 8) % NT == 0 || tid + i * NT < BN * 8) *reinterpret_cast<u32x4*>(smem + buf * STAGE + BM * BK + wdst[i]) = wreg[i];
    }
  };

  // ---- fragment addressing: lane l reads row (l%16), 16-byte chunk kk*4 + l/16
  const int frow = lane & 15;
  const int fchk = lane >> 4;

  f32x4 acc[TM][TN];
  uint32_t t[TM][TN][2];                 // current node, packed bf16 (n, n+1), (n+2, n+3)
  uint32_t s0[TM][TN][2];                // level 0: running left-to-right sum
  uint32_t sb[LBMAX > 0 ? LBMAX : 1][TM][TN][2];  // binary levels
  int c0 = 0;                            // leaves absorbed at level 0
  int g = 0;                             // groups completed (binary counter)

  const int nstages = TREE ? p.T * LS : (p.K + BK - 1) / BK;
  const int nouter = TREE ? p.T : (nstages + LS - 1) / LS;

  load_stage(0, 0);
  if (NSET == 2) load_stage(min(1, nstages - 1), 1);
  store_stage(0, 0);
  __syncthreads();

  for (int j = 0; j < nouter; j++) {
#pragma unroll
    for (int i = 0; i < LS; i++) {
      const int s = j * LS + i;
      if (TREE || s < nstages) {
        // the stage after the last one re-reads the last one into the idle buffer: harmless, and it
        // keeps the staging registers free of control flow
        if (NSET == 1) load_stage(min(s + 1, nstages - 1), 0);
        else load_stage(min(s + 2, nstages - 1), i & 1);  // the set that held stage s, stored a stage ago
        const uint16_t* bx = smem + (s & 1) * STAGE;
        const uint16_t* bw = bx + BM * BK;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
          bf16x8 fx[TM], fw[TN];
#pragma unroll
          for (int a = 0; a < TM; a++) {
            const int r = (wm * TM + a) * 16 + frow;
            fx[a] = *reinterpret_cast<const bf16x8*>(bx + lds_off(r, kk * 4 + fchk));
          }
#pragma unroll
          for (int b = 0; b < TN; b++) {
            const int r = (wn * TN + b) * 16 + frow;
            fw[b] = *reinterpret_cast<const bf16x8*>(bw + lds_off(r, kk * 4 + fchk));
          }
          const bool fresh = (i == 0 && kk == 0) && (TREE || j == 0);
#pragma unroll
          for (int a = 0; a < TM; a++)
#pragma unroll
            for (int b = 0; b < TN; b++) {
              const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
              acc[a][b] = Num::mfma(fw[b], fx[a], fresh ? zero : acc[a][b]);
            }
        }
        store_stage((s + 1) & 1, NSET == 1 ? 0 : (i + 1) & 1);
        __syncthreads();
      }
    }
    if (TREE) {
      // leaf -> bf16, then the binary-counter merge (all conditions are uniform over the block)
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++) {
          t[a][b][0] = Num::pack(acc[a][b][0], acc[a][b][1]);
          t[a][b][1] = Num::pack(acc[a][b][2], acc[a][b][3]);
        }
      if (c0 != 0) {
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
          for (int b = 0; b < TN; b++) {
            t[a][b][0] = Num::add(s0[a][b][0], t[a][b][0]);
            t[a][b][1] = Num::add(s0[a][b][1], t[a][b][1]);
          }
      }
      c0++;
      if (c0 == p.flb) {
        c0 = 0;
        bool parked = false;
#pragma unroll
        for (int l = 0; l < LBMAX; l++) {
          if (!parked && l < p.lb) {
            if ((g >> l) & 1) {
#pragma unroll
              for (int a = 0; a < TM; a++)
#pragma unroll
                for (int b = 0; b < TN; b++) {
                  t[a][b][0] = Num::add(sb[l][a][b][0], t[a][b][0]);
                  t[a][b][1] = Num::add(sb[l][a][b][1], t[a][b][1]);
                }
            } else {
#pragma unroll
              for (int a = 0; a < TM; a++)
#pragma unroll
                for (int b = 0; b < TN; b++) {
                  sb[l][a][b][0] = t[a][b][0];
                  sb[l][a][b][1] = t[a][b][1];
                }
              parked = true;
            }
          }
        }
        g++;
      } else {
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
          for (int b = 0; b < TN; b++) {
            s0[a][b][0] = t[a][b][0];
            s0[a][b][1] = t[a][b][1];
          }
      }
    }
  }

  // ---- epilogue: (bias in fp32 for the single-accumulator GEMM, in bf16 after the tree), store
#pragma unroll
  for (int a = 0; a < TM; a++) {
    const int m = m0 + (wm * TM + a) * 16 + frow;
#pragma unroll
    for (int b = 0; b < TN; b++) {
      const int n = n0 + (wn * TN + b) * 16 + fchk * 4;
      if (m >= p.M || n >= p.N) continue;
      uint32_t lo, hi;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) {
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (n + e < p.N) bv[e] = Num::to_f32(p.bias[n + e]);
      }
      if (TREE) {
        lo = t[a][b][0];
        hi = t[a][b][1];
        if (p.bias) {
          lo = Num::add(lo, Num::pack(bv[0], bv[1]));
          hi = Num::add(hi, Num::pack(bv[2], bv[3]));
        }
      } else {
        lo = Num::pack(acc[a][b][0] + bv[0], acc[a][b][1] + bv[1]);
        hi = Num::pack(acc[a][b][2] + bv[2], acc[a][b][3] + bv[3]);
      }
      uint16_t* dst = Cs + (int64_t)m * p.ldc + n;
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

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
template <int WAVES_M, int WAVES_N, int TM, int TN, int LS, int LBMAX, bool TREE, bool F16, bool WT = false>
static int launch(const GemmArgs& a, int split, hipStream_t stream) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * TM * 16;
  constexpr int BN = WAVES_N * TN * 16;
  constexpr size_t smem = (size_t)2 * (BM + BN) * BK * sizeof(uint16_t);
  auto kern = gemm_kernel<WAVES_M, WAVES_N, TM, TN, LS, LBMAX, TREE, F16, WT>;
  if (smem > 48 * 1024) {
    static std::atomic<uint64_t> done{0};
    hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), (int)smem, done);
    if (e != hipSuccess) return hip_code(e);
  }
  const int64_t tiles = (int64_t)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  if (tiles <= 0 || tiles > 0x7fffffff) return TBIK_ERR_INVALID;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)split), dim3(NT), smem, stream, a);
  return hip_code(hipGetLastError());
}

template <int LS, int LBMAX, bool TREE, bool F16>
static int launch_by_m(const GemmArgs& a, int split, hipStream_t stream) {
  if (a.M <= 16) return launch<1, 4, 1, 1, LS, LBMAX, TREE, F16>(a, split, stream);
  if (a.M <= 64) return launch<1, 4, 4, 2, LS, LBMAX, TREE, F16>(a, split, stream);
  // without a split over K (the single-accumulator mm) a small grid of 128x128 tiles leaves CUs idle: 64x128 tiles
  // double the work-groups (the choice cannot change any bit: the chain per element is the same)
  if (!TREE && (int64_t)((a.M + 127) / 128) * ((a.N + 127) / 128) < 256) {
    if ((int64_t)((a.M + 63) / 64) * ((a.N + 127) / 128) < 256) return launch<1, 4, 4, 1, LS, LBMAX, TREE, F16>(a, split, stream);
    return launch<1, 4, 4, 2, LS, LBMAX, TREE, F16>(a, split, stream);
  }
  return launch<2, 2, 4, 4, LS, LBMAX, TREE, F16>(a, split, stream);
}

// Row-major B[K,N]: two tile shapes (16 and 64 rows), the deepest merge stack
template <int LS, int LBMAX, bool TREE, bool F16>
static int launch_rowmajor_b(const GemmArgs& a, int split, hipStream_t stream) {
  if (a.M <= 16) return launch<1, 4, 1, 1, LS, LBMAX, TREE, F16, true>(a, split, stream);
  return launch<1, 4, 4, 2, LS, LBMAX, TREE, F16, true>(a, split, stream);
}

template <int LS, bool F16>
static int launch_tree(const GemmArgs& a, int split, hipStream_t stream) {
  if (a.lb <= 2) return launch_by_m<LS, 2, true, F16>(a, split, stream);
  if (a.lb <= 4) return launch_by_m<LS, 4, true, F16>(a, split, stream);
  if (a.lb <= 6) return launch_by_m<LS, 6, true, F16>(a, split, stream);
  return TBIK_ERR_UNSUPPORTED;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// How one problem is run.  Small grids are filled by cutting K into `split` aligned subtrees (one grid.y slice
// each) whose bf16 partials meet in the shard tree afterwards -- the same arithmetic as tensor-parallel shards, so
// the bits do not change.  The wide kernel takes over once its 128x256 tiles (times the split) occupy the chip.
struct Plan {
  bool wide;
  int split;       // power of two, divides 2^lb
  int T, flb, lb;  // tree of ONE shard
  size_t partial_bytes, parked_bytes;
};

// Which of the two 128x256-tile kernels runs a shard whose tree has groups of `flb` leaves and `lb` binary levels.  The
// kernel that keeps two binary levels in registers parks and re-reads a level less than half as often, which pays when
// levels are parked often: groups of two leaves from two levels on (13 % at K = 8192), any tree from four levels on;
// on the other trees its branchy loop body loses about 3 %.  (bf16 only: an fp16 node is a single packed add, so there
// is little to save.)
static bool wide_uses_deep_kernel(int leaf_k, bool f16, int flb, int lb) {
  return leaf_k == 256 && !f16 && (lb >= 4 || (flb == 2 && lb >= 2));
}

// Estimated time of the 128x256-tile kernels over the legal K splits of one problem, and the best split: rounds of
// work-groups on 256 CUs, each round a fixed part (pipeline fill, last merges, store) plus the K extent of one shard at
// the rate of the kernel that shard would run on, plus the shard-combine pass over (split + 1) [M,N] arrays.  Constants
// measured on MI355X: 5.5 us per round; 16.5 ns per k (15.0 on the kernel for deep trees); 5 TB/s and 4 us for the
// combine.
static double wide_cost_us(int M, int N, int K, int leaf_k, bool f16, int flb, int lb, int* best_split) {
  const int max_split = lb >= 5 ? 32 : (1 << lb);
  const int64_t wide_tiles = (int64_t)((M + 127) / 128) * ((N + 255) / 256);
  double best = 0;
  int split = 1, ls = 0;
  for (int sp = 1; sp <= max_split; sp *= 2, ls++) {
    if (sp > 8 && wide_tiles * sp > 256) break;  // finer cuts only while the whole grid still runs as one round
    const double rounds = (double)((wide_tiles * sp + 255) / 256);
    const double ns_per_k = wide_uses_deep_kernel(leaf_k, f16, flb, lb - ls) ? 0.0150 : 0.0165;
    double t = rounds * (5.5 + ((double)K / sp) * ns_per_k);
    if (sp > 1) t += 4.0 + (double)(sp + 1) * M * N * 2.0 / 5.0e6;
    if (sp == 1 || t < best) {
      best = t;
      split = sp;
    }
  }
  *best_split = split;
  return best;
}

// Column regions.  A grid of 128x256 tiles rarely fills whole rounds of 256 work-groups, and one K split serves the
// whole problem; cut into the columns [0, NA) and [NA, N), each part gets the split that fills ITS rounds (o_proj 32B
// at M=4096: 512 tiles unsplit = two full rounds, then 128 tiles cut in two = one round of half the length, instead of
// three rounds: 395 -> 350 us; at M=512: 64 tiles cut in four and 16 tiles cut in sixteen, 74 -> 69 us).  The parts
// run one after the other as problems of their own, so every element is still computed by the same leaf and shard
// trees: the bits do not change.  Returns NA (a multiple of 256), or 0 when the whole problem in one piece is
// estimated within 5 % of the best pair.
static int column_regions(int M, int N, int K, int leaf_k, bool f16) {
  int T, flb, level_k;
  if (M < 64 || N <= 256 || tbik_tree_params(K, leaf_k, &T, &flb, &level_k) != TBIK_OK) return 0;
  const int tiles_n = (N + 255) / 256;
  if (tiles_n > 64) return 0;
  int sp;
  const double whole = wide_cost_us(M, N, K, leaf_k, f16, flb, level_k - 1, &sp);
  double best = whole * 0.95;
  int best_na = 0;
  for (int na = 1; na < tiles_n; na++) {
    const double t = wide_cost_us(M, na * 256, K, leaf_k, f16, flb, level_k - 1, &sp) +
                     wide_cost_us(M, N - na * 256, K, leaf_k, f16, flb, level_k - 1, &sp);
    if (t < best) {
      best = t;
      best_na = na * 256;
    }
  }
  return best_na;
}

static bool make_plan(int M, int N, int K, int leaf_k, bool f16, Plan* pl, bool rowmajor_b = false) {
  int T, flb, level_k;
  if (M <= 0 || N <= 0 || tbik_tree_params(K, leaf_k, &T, &flb, &level_k) != TBIK_OK) return false;
  const int lb = level_k - 1;
  const int max_split = lb >= 5 ? 32 : (1 << lb);
  const int64_t wide_tiles = (int64_t)((M + 127) / 128) * ((N + 255) / 256);
  int split = 1;
  bool wide = false;
  if (M >= 64 && !rowmajor_b) {  // the wide kernels exist for [N,K] weights only
    wide_cost_us(M, N, K, leaf_k, f16, flb, lb, &split);
    // exactly 64 rows fit one 64-row tile of the tiled kernel, which half-empty 128-row tiles only beat on a grid that
    // fills most of the chip: [64,25600] x [25600,4096] 66 us on 128 work-groups of the wide kernel, 51 on the tiled one;
    // [64,16384] x [16384,8192] 75 on 256 against 97
    wide = wide_tiles * split >= (M == 64 ? 160 : 64);
  }
  if (!wide) {
    const int bm = M <= 16 ? 16 : ((M <= 64 || rowmajor_b) ? 64 : 128), bn = M <= 16 ? 64 : 128;
    const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    split = 1;
    while (tiles * split < 512 && split < max_split && split < 8) split *= 2;
  }
  int ls = 0;
  while ((1 << ls) < split) ls++;
  pl->wide = wide;
  pl->split = split;
  pl->T = T / split;
  pl->flb = flb;
  pl->lb = lb - ls;
  pl->partial_bytes = split > 1 ? (size_t)split * M * N * sizeof(uint16_t) : 0;
  pl->partial_bytes = (pl->partial_bytes + 255) & ~(size_t)255;
  pl->parked_bytes = wide ? wide_workspace_bytes(M, N, pl->lb, split, wide_uses_deep_kernel(leaf_k, f16, flb, pl->lb) ? 2 : 1) : 0;
  return true;
}

// 64 .. 512 rows, leaves of 256: one to four rows of 128x256 tiles need a deep cut of K to occupy the chip, and the pass
// over that many partial results then weighs as much as a quarter of the GEMM.  Tiles of 128 columns
// (gemm_tree_quad.hip) occupy it with half the cut.  That kernel is slower per slice than the 128x256-tile kernels, so it
// is taken only where a shard is short and the grid close to one work-group per CU, the region where sweeps over
// N = 1024 .. 8192 and K = 2048 .. 16384 on MI355X measured it ahead:
//   * 64 .. 128 rows (one row of tiles): shards of 512 .. 1024 of K on 160 .. 256 work-groups, or up to 1536 on
//     224 .. 256 -- 8 % on average, up to 20 %; with fewer rows the 64-row tiles of the tiled kernel win;
//   * 129 .. 512 rows (two to four rows of tiles): only shards of at most 1024 and a cut into at least four -- 6 % on
//     average, ahead in every one of 59 shapes in three alternating repetitions each.
// The shards are aligned subtrees like every other K split, so the bits do not change.
struct NarrowPlan {
  int split;
  int T, flb, lb;  // tree of ONE shard
  size_t partial_bytes;
};

static bool narrow_plan(int M, int N, int K, int leaf_k, bool f16, NarrowPlan* np) {
  int T, flb, level_k;
  if (f16 || leaf_k != 256 || M < 64 || M > 512 || tbik_tree_params(K, leaf_k, &T, &flb, &level_k) != TBIK_OK) return false;
  // exactly 64 rows: the 64-row tiles of the tiled kernel cut K at most eightfold, which fills the chip from 32 column
  // tiles on and then beats 128-row tiles that are half empty ([64,8192] x [8192,4096] 25.6 -> 21.1 us, [64,4096] x
  // [4096,4096] 14.7 -> 13.5); narrower matrices need the deeper cut of this plan (N = 2048: 15.5 against 16.8)
  if (M == 64 && N >= 4096) return false;
  const int lb = level_k - 1;
  const int64_t tiles = (((int64_t)N + 127) / 128) * ((M + 127) / 128);
  int best = 0, best_ls = 0;
  int64_t best_wgs = 0;
  for (int ls = 0; ls <= lb && ls <= 5; ls++) {
    const int sp = 1 << ls;
    const int ks = K / sp;
    const int64_t wgs = tiles * sp;
    if (lb - ls > 1 || ks < 512 || ks > 1536 || wgs > 256 || wgs < (ks > 1024 ? 224 : 160)) continue;
    if (M > 128 && (sp < 4 || ks > 1024)) continue;
    if (wgs > best_wgs) {
      best_wgs = wgs;
      best = sp;
      best_ls = ls;
    }
  }
  if (!best) return false;
  np->split = best;
  np->T = T / best;
  np->flb = flb;
  np->lb = lb - best_ls;
  np->partial_bytes = best > 1 ? (((size_t)best * M * N * sizeof(uint16_t) + 255) & ~(size_t)255) : 0;
  return true;
}

// The two column regions of a problem (column_regions): when both run on the same 128x256-tile kernel they go out as
// ONE launch (the short work-groups of one region fill the CUs that the long ones of the other leave early) and each
// needs a workspace of its own; otherwise they run one after the other and share it.
struct RegionPlan {
  int na;     // columns of the first region; 0: the problem runs in one piece
  bool pair;  // one launch for both
  Plan a, b;
  bool narrow_a, narrow_b;  // the region runs on 128x128 tiles (narrow_plan) instead of plan a / b
  size_t bytes_a, bytes_b, bytes;
};

// How a tree GEMM runs.  tree_plan() is the ONE place that decides it: the workspace query and the dispatcher both call
// it, so the bytes the caller is told to bring are the bytes the launch uses.
enum TreePath {
  PATH_STRIP = 0,    // a few rows: one launch, K cut over the waves of a work-group, no workspace
  PATH_NARROW = 1,   // 64 .. 512 rows, short shards: 128x128 tiles (narrow_plan)
  PATH_REGIONS = 2,  // two column regions, each with a K split of its own (column_regions)
  PATH_SINGLE = 3,   // one grid of 128x256 tiles or of the small tiles, one K split (make_plan)
};
struct TreePlan {
  TreePath path;
  int strip_waves;     // PATH_STRIP
  NarrowPlan narrow;   // PATH_NARROW
  RegionPlan regions;  // PATH_REGIONS
  Plan single;         // PATH_SINGLE
  size_t bytes;        // workspace of the chosen path
};

static bool tree_plan(int M, int N, int K, int leaf_k, bool f16, bool rowmajor_b, bool whole_problem, TreePlan* tp);

static bool plan_regions(int M, int N, int K, int leaf_k, bool f16, RegionPlan* rp) {
  rp->na = column_regions(M, N, K, leaf_k, f16);
  if (!rp->na) return false;
  // each region is planned as a problem of its own (never cut again): what it needs is what its launch will use
  TreePlan ta, tb;
  if (!tree_plan(M, rp->na, K, leaf_k, f16, false, false, &ta) || !tree_plan(M, N - rp->na, K, leaf_k, f16, false, false, &tb) ||
      ta.path == PATH_STRIP || tb.path == PATH_STRIP) {
    rp->na = 0;
    return false;
  }
  // a region that qualifies for the 128x128 tiles takes them (o_proj 32B at M=512: the 1024 columns cut into sixteen
  // become 32 tiles cut into eight)
  rp->narrow_a = ta.path == PATH_NARROW;
  rp->narrow_b = tb.path == PATH_NARROW;
  if (!make_plan(M, rp->na, K, leaf_k, f16, &rp->a) || !make_plan(M, N - rp->na, K, leaf_k, f16, &rp->b)) {
    rp->na = 0;
    return false;
  }
  rp->bytes_a = (ta.bytes + 255) & ~(size_t)255;
  rp->bytes_b = (tb.bytes + 255) & ~(size_t)255;
  rp->pair = !rp->narrow_a && !rp->narrow_b && rp->a.wide && rp->b.wide &&
             wide_uses_deep_kernel(leaf_k, f16, rp->a.flb, rp->a.lb) == wide_uses_deep_kernel(leaf_k, f16, rp->b.flb, rp->b.lb);
  rp->bytes = rp->pair ? rp->bytes_a + rp->bytes_b : std::max(rp->bytes_a, rp->bytes_b);
  return true;
}

// whole_problem: the call may still be cut into column regions (false for a region itself).  Returns false for shapes
// no tree exists for (K not a whole number of leaves).
static bool tree_plan(int M, int N, int K, int leaf_k, bool f16, bool rowmajor_b, bool whole_problem, TreePlan* tp) {
  int T, flb, level_k;
  if (M <= 0 || N <= 0 || tbik_tree_params(K, leaf_k, &T, &flb, &level_k) != TBIK_OK) return false;
  tp->bytes = 0;
  tp->strip_waves = 0;
  if (!rowmajor_b) {
    tp->strip_waves = gemm_tree_strip_waves(M, N, K, level_k - 1);
    if (tp->strip_waves) {
      tp->path = PATH_STRIP;
      return true;
    }
    if (narrow_plan(M, N, K, leaf_k, f16, &tp->narrow)) {
      tp->path = PATH_NARROW;
      tp->bytes = tp->narrow.partial_bytes;
      return true;
    }
    if (whole_problem && plan_regions(M, N, K, leaf_k, f16, &tp->regions)) {
      tp->path = PATH_REGIONS;
      tp->bytes = tp->regions.bytes;
      return true;
    }
  }
  if (!make_plan(M, N, K, leaf_k, f16, &tp->single, rowmajor_b)) return false;
  tp->path = PATH_SINGLE;
  tp->bytes = tp->single.partial_bytes + tp->single.parked_bytes;
  return true;
}

size_t gemm_workspace_bytes(int M, int N, int K, int leaf_k, bool f16, bool rowmajor_b) {
  TreePlan tp;
  return tree_plan(M, N, K, leaf_k, f16, rowmajor_b, true, &tp) ? tp.bytes : 0;
}

// What tree_plan() chose for a shape, for callers and tests that want to know (no effect on any result):
// out[0] path (0 one-launch few-rows kernel, 1 128x128 tiles, 2 two column regions, 3 one grid), out[1] K split (of the
// first region for path 2; waves per strip for path 0), out[2] columns of the first region (path 2, else 0), out[3] K
// split of the second region (path 2, else 0), out[4] 1 when the two regions go out as one launch.
int gemm_plan_info(int M, int N, int K, int leaf_k, bool f16, bool rowmajor_b, int out[5]) {
  TreePlan tp;
  if (!out) return TBIK_ERR_INVALID;
  if (!tree_plan(M, N, K, leaf_k, f16, rowmajor_b, true, &tp)) return TBIK_ERR_INVALID;
  out[0] = (int)tp.path;
  out[1] = tp.path == PATH_STRIP ? tp.strip_waves : tp.path == PATH_NARROW ? tp.narrow.split
           : tp.path == PATH_REGIONS ? (tp.regions.narrow_a ? 0 : tp.regions.a.split) : tp.single.split;
  out[2] = tp.path == PATH_REGIONS ? tp.regions.na : 0;
  out[3] = tp.path == PATH_REGIONS ? (tp.regions.narrow_b ? 0 : tp.regions.b.split) : 0;
  out[4] = tp.path == PATH_REGIONS && tp.regions.pair ? 1 : 0;
  return TBIK_OK;
}

static int gemm_dispatch_impl(bool tree, bool f16, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n,
                              void* C, int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, void* ws,
                              size_t ws_bytes, hipStream_t stream, bool whole_problem, const NormEpilogue* ep = nullptr);

int gemm_dispatch(bool tree, bool f16, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                  int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, void* ws, size_t ws_bytes,
                  hipStream_t stream) {
  return gemm_dispatch_impl(tree, f16, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, leaf_k, bias, ws, ws_bytes, stream, true);
}

// The tree matmul with the (add-)RMSNorm of its result inside the launch of its shard combine: `out` receives the
// normalised rows, res_out the result + residual.  TBIK_ERR_UNSUPPORTED (nothing launched) where the matmul of this shape
// has no shard combine over whole rows; the caller then runs the matmul and the norm as two calls.  Same bits either way.
int gemm_tree_rmsnorm_dispatch(bool f16, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, int M, int N,
                               int K, int leaf_k, const void* bias, const void* res, int64_t ldr, const void* norm_w, float eps,
                               void* res_out, int64_t ldro, void* out, int64_t ldo, void* ws, size_t ws_bytes,
                               hipStream_t stream) {
  if (res && !res_out) return TBIK_ERR_INVALID;
  if (M <= 0 || N <= 0) return TBIK_ERR_UNSUPPORTED;
  auto bad = [](const void* p, int64_t ld) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0 || (ld & 7) != 0; };
  if ((res && (bad(res, ldr) || bad(res_out, ldro) || ldr < N || ldro < N)) || (norm_w && bad(norm_w, 8))) return TBIK_ERR_ALIGNMENT;
  const NormEpilogue ep{res, ldr, norm_w, eps, res ? res_out : nullptr, ldro};
  return gemm_dispatch_impl(true, f16, A, lda, B, ldb_k, ldb_n, out, ldo, M, N, K, leaf_k, bias, ws, ws_bytes, stream, true, &ep);
}

static int gemm_dispatch_impl(bool tree, bool f16, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n,
                              void* C, int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, void* ws,
                              size_t ws_bytes, hipStream_t stream, bool whole_problem, const NormEpilogue* ep) {
  if (M < 0 || N < 0 || K <= 0) return TBIK_ERR_INVALID;
  if (M == 0 || N == 0) return TBIK_OK;  // nothing to do (empty tensors may come with null pointers)
  if (!A || !B || !C) return TBIK_ERR_INVALID;
  // B[K,N] row-major (ldb_n == 1) is consumed in place by the tiled kernels; [N,K] K-contiguous (ldb_k == 1, the
  // nn.Linear weight) is the native layout of all of them
  const bool rowmajor_b = ldb_k != 1;
  if (rowmajor_b && ldb_n != 1) return TBIK_ERR_UNSUPPORTED;  // neither dimension contiguous
  const int64_t ldw = rowmajor_b ? ldb_k : ldb_n;
  if (lda < K || ldw < (rowmajor_b ? N : K) || ldc < N) return TBIK_ERR_INVALID;
  if (!aligned16(A) || !aligned16(B) || (lda & 7) || (ldw & 7) || (K & 7)) return TBIK_ERR_ALIGNMENT;
  if (reinterpret_cast<uintptr_t>(C) & 1) return TBIK_ERR_ALIGNMENT;

  GemmArgs a;
  a.X = static_cast<const uint16_t*>(A);
  a.W = static_cast<const uint16_t*>(B);
  a.C = static_cast<uint16_t*>(C);
  a.bias = static_cast<const uint16_t*>(bias);
  a.ldx = lda;
  a.ldw = ldw;
  a.ldc = ldc;
  a.M = M;
  a.N = N;
  a.K = K;
  a.T = 0;
  a.flb = 1;
  a.lb = 0;
  a.vec_store = ((reinterpret_cast<uintptr_t>(C) & 7) == 0 && (ldc & 3) == 0) ? 1 : 0;
  a.k_shard = 0;
  a.c_shard = 0;
  if (!tree && rowmajor_b)
    return f16 ? launch_rowmajor_b<4, 0, false, true>(a, 1, stream) : launch_rowmajor_b<4, 0, false, false>(a, 1, stream);
  if (!tree) {
    // large problems whose K is a whole number of 64-wide slices take the one-wave-per-SIMD pipeline (same MFMA
    // chain per element, so the same bits as the tiled kernel)
    const int64_t wide_tiles = (int64_t)((M + 127) / 128) * ((N + 255) / 256);
    // 33..128 rows: one row of 128-row tiles whose width balances the grid, when such a grid exists (same MFMA chain
    // per element again; measured faster than the streaming kernel from 33 rows on)
    const bool narrow_n = N < 4096;   // no one-row grid of at least 128 tiles, whatever their width
    if (!f16 && M > 32 && M <= 128 && (K & 63) == 0 && lda < (1 << 22) && ldb_n < (1 << 22)) {
      QuadArgs qa{a.X, a.W, a.C, a.bias, a.ldx, a.ldw, a.ldc, M, N, K, a.vec_store};
      if (!narrow_n) {
        const int rc = gemm_single_acc_slab_launch(qa, stream);
        if (rc != TBIK_ERR_UNSUPPORTED) return rc;
      } else {
        // a narrow weight matrix (a TP shard of a column-split layer): the width chosen by the cost model of the larger
        // batches beats the streaming kernel (too few strips to fill the chip) and the tiled one from 33 rows on --
        // [M,4096]x[4096,768] 25 -> 16 us at 33-48 rows, 41 -> 17-22 at 65-128; [M,6144]x[6144,2048] 37 -> 23 and
        // 59 -> 26-34; [M,12288]x[12288,1536] 70 -> 42 and 115 -> 47-63 (up to 24 rows the streaming kernel still wins)
        return gemm_single_acc_balanced_launch(qa, stream);
      }
    }
    // more rows: the same pipeline with the tile width that spreads the grid over the chip (128x256 on large shapes)
    if (!f16 && M > 128 && (K & 63) == 0 && lda < (1 << 22) && ldb_n < (1 << 22)) {
      QuadArgs qa{a.X, a.W, a.C, a.bias, a.ldx, a.ldw, a.ldc, M, N, K, a.vec_store};
      return gemm_single_acc_balanced_launch(qa, stream);
    }
    if (!f16 && M > 64 && wide_tiles >= 128 && (K & 63) == 0 && lda < (1 << 22) && ldb_n < (1 << 22)) {
      QuadArgs qa{a.X, a.W, a.C, a.bias, a.ldx, a.ldw, a.ldc, M, N, K, a.vec_store};
      return gemm_single_acc_quad_launch(qa, stream);
    }
    // a handful of rows: one pass over the weights, every 16x16 tile its own wave (same chain per element again)
    if (M <= 64 && (K & 31) == 0) {
      StreamArgs sa{a.X, a.W, a.C, a.bias, a.ldx, a.ldw, a.ldc, M, N, K, a.vec_store};
      return gemm_single_acc_stream_launch(sa, f16, stream);
    }
    return f16 ? launch_by_m<4, 0, false, true>(a, 1, stream) : launch_by_m<4, 0, false, false>(a, 1, stream);
  }

  if (leaf_k != 256 && leaf_k != 128) return TBIK_ERR_UNSUPPORTED;
  TreePlan tp;
  if (!tree_plan(M, N, K, leaf_k, f16, rowmajor_b, whole_problem, &tp)) return TBIK_ERR_INVALID;
  if (ep) {
    // the norm rides on the shard combine of ONE K split over all columns: nothing else has a pass over whole rows
    const bool combines = (tp.path == PATH_NARROW && tp.narrow.split > 1) || (tp.path == PATH_SINGLE && tp.single.split > 1);
    if (!combines || N > 16 * 512 || (N & 7) || !aligned16(C) || (ldc & 7)) return TBIK_ERR_UNSUPPORTED;
  }
  auto combine = [&](const void* const* parts, int nparts) {
    if (ep)
      return tree_combine_rmsnorm_dispatch(parts, nparts, M, N, bias, ep->res, ep->ldr, ep->w, ep->eps, C, ldc, ep->res_out,
                                           ep->ldro, nullptr, 0, f16, stream);
    // one launch adds the shards (and the bias) in tree order, into C's own row stride
    return tree_combine_bias_dispatch(parts, nparts, C, (int64_t)M * N, bias, N, f16, stream, ldc);
  };
  if (tp.path == PATH_STRIP) {
    // a handful of rows: one launch, K cut over the waves of a work-group, nothing goes through the workspace
    int T, flb, level_k;
    tbik_tree_params(K, leaf_k, &T, &flb, &level_k);
    StripArgs sa{a.X, a.W, a.C, a.bias, a.ldx, a.ldw, a.ldc, M, N, K, flb, level_k - 1, a.vec_store};
    return gemm_tree_strip_launch(sa, leaf_k, tp.strip_waves, f16, stream);
  }
  if (tp.path == PATH_NARROW) {
    const NarrowPlan& np = tp.narrow;
    if (np.partial_bytes > 0 && (!ws || ws_bytes < np.partial_bytes || !aligned16(ws))) return TBIK_ERR_WORKSPACE;
    WideArgs w{a.X, a.W, a.C, a.bias, nullptr, a.ldx, a.ldw, a.ldc, M, N, K / np.split, np.T, np.flb, np.lb, a.vec_store,
               (int64_t)(K / np.split), 0};
    if (np.split > 1) {
      w.C = static_cast<uint16_t*>(ws);
      w.ldc = N;
      w.c_shard = (int64_t)M * N;
      w.vec_store = (N & 3) == 0 ? 1 : 0;
      w.bias = nullptr;
    }
    const int rc = gemm_tree_quad_launch(w, np.split, stream);
    if (rc != TBIK_OK || np.split == 1) return rc;
    const void* parts[32];
    for (int i = 0; i < np.split; i++) parts[i] = static_cast<uint8_t*>(ws) + (size_t)i * M * N * sizeof(uint16_t);
    return combine(parts, np.split);
  }
  if (tp.path == PATH_REGIONS) {
    const RegionPlan& rp = tp.regions;
    const size_t esz = sizeof(uint16_t);
    const int na = rp.na;
    const void* Bb = static_cast<const uint8_t*>(B) + (size_t)na * ldb_n * esz;
    void* Cb = static_cast<uint8_t*>(C) + (size_t)na * esz;
    const void* bias_b = bias ? static_cast<const uint8_t*>(bias) + (size_t)na * esz : nullptr;
    if (!rp.pair) {
      // columns [0, na) and [na, N) as problems of their own, one after the other on the stream, sharing the workspace
      const int rc = gemm_dispatch_impl(tree, f16, A, lda, B, ldb_k, ldb_n, C, ldc, M, na, K, leaf_k, bias, ws, ws_bytes,
                                        stream, false);
      if (rc != TBIK_OK) return rc;
      return gemm_dispatch_impl(tree, f16, A, lda, Bb, ldb_k, ldb_n, Cb, ldc, M, N - na, K, leaf_k, bias_b, ws, ws_bytes,
                                stream, false);
    }
    if (rp.bytes > 0 && (!ws || ws_bytes < rp.bytes || !aligned16(ws))) return TBIK_ERR_WORKSPACE;
    uint8_t* wsa = static_cast<uint8_t*>(ws);
    uint8_t* wsb2 = wsa + rp.bytes_a;
    // the kernel arguments of one region: its shards write [M, n] partials into its workspace when K is cut
    auto region_args = [&](const Plan& pl, const void* Bw, void* Cr, const void* bias_r, int n, uint8_t* w) {
      WideArgs r{a.X, static_cast<const uint16_t*>(Bw), static_cast<uint16_t*>(Cr), static_cast<const uint16_t*>(bias_r),
                 reinterpret_cast<u32x4*>(w + pl.partial_bytes), a.ldx, a.ldw, a.ldc, M, n, K / pl.split, pl.T, pl.flb, pl.lb,
                 ((reinterpret_cast<uintptr_t>(Cr) & 7) == 0 && (ldc & 3) == 0) ? 1 : 0, (int64_t)(K / pl.split), 0};
      if (pl.split > 1) {
        r.C = reinterpret_cast<uint16_t*>(w);
        r.ldc = n;
        r.c_shard = (int64_t)M * n;
        r.vec_store = (n & 3) == 0 ? 1 : 0;
        r.bias = nullptr;
      }
      return r;
    };
    const WideArgs ra = region_args(rp.a, B, C, bias, na, wsa);
    const WideArgs rb = region_args(rp.b, Bb, Cb, bias_b, N - na, wsb2);
    // the region with the longer shards first
    const bool a_first = ra.K >= rb.K;
    const WidePair pair{a_first ? ra : rb, a_first ? rb : ra, a_first ? rp.a.split : rp.b.split, a_first ? rp.b.split : rp.a.split};
    int rc = wide_uses_deep_kernel(leaf_k, f16, rp.a.flb, rp.a.lb) ? gemm_tree_deep_pair_launch(pair, stream)
                                                                   : gemm_tree_wide_pair_launch(pair, leaf_k, f16, stream);
    if (rc != TBIK_OK) return rc;
    const void* parts[32];
    if (rp.a.split > 1) {
      for (int i = 0; i < rp.a.split; i++) parts[i] = wsa + (size_t)i * M * na * esz;
      rc = tree_combine_bias_dispatch(parts, rp.a.split, C, (int64_t)M * na, bias, na, f16, stream, ldc);
      if (rc != TBIK_OK) return rc;
    }
    if (rp.b.split > 1) {
      for (int i = 0; i < rp.b.split; i++) parts[i] = wsb2 + (size_t)i * M * (N - na) * esz;
      rc = tree_combine_bias_dispatch(parts, rp.b.split, Cb, (int64_t)M * (N - na), bias_b, N - na, f16, stream, ldc);
    }
    return rc;
  }
  const Plan& pl = tp.single;
  if (tp.bytes > 0 && (!ws || ws_bytes < tp.bytes || !aligned16(ws))) return TBIK_ERR_WORKSPACE;
  uint8_t* wsb = static_cast<uint8_t*>(ws);
  a.T = pl.T;
  a.flb = pl.flb;
  a.lb = pl.lb;
  a.k_shard = K / pl.split;
  a.K = K / pl.split;
  if (pl.split > 1) {
    // shards write contiguous [M,N] partials into the workspace; bias is applied after the shard tree
    a.C = reinterpret_cast<uint16_t*>(wsb);
    a.ldc = N;
    a.c_shard = (int64_t)M * N;
    a.vec_store = (N & 3) == 0 ? 1 : 0;
    a.bias = nullptr;
  }
  int rc;
  if (rowmajor_b) {
    if (a.lb > 6) return TBIK_ERR_UNSUPPORTED;
    if (f16) rc = leaf_k == 256 ? launch_rowmajor_b<4, 6, true, true>(a, pl.split, stream) : launch_rowmajor_b<2, 6, true, true>(a, pl.split, stream);
    else rc = leaf_k == 256 ? launch_rowmajor_b<4, 6, true, false>(a, pl.split, stream) : launch_rowmajor_b<2, 6, true, false>(a, pl.split, stream);
  } else if (pl.wide) {
    WideArgs w{a.X, a.W, a.C, a.bias, reinterpret_cast<u32x4*>(wsb + pl.partial_bytes), a.ldx, a.ldw, a.ldc, M, N, a.K,
               a.T, a.flb, a.lb, a.vec_store, a.k_shard, a.c_shard};
    rc = wide_uses_deep_kernel(leaf_k, f16, a.flb, a.lb) ? gemm_tree_deep_launch(w, pl.split, stream)
                                                         : gemm_tree_wide_launch(w, leaf_k, f16, pl.split, stream);
  } else {
    if (f16) rc = leaf_k == 256 ? launch_tree<4, true>(a, pl.split, stream) : launch_tree<2, true>(a, pl.split, stream);
    else rc = leaf_k == 256 ? launch_tree<4, false>(a, pl.split, stream) : launch_tree<2, false>(a, pl.split, stream);
  }
  if (rc != TBIK_OK || pl.split == 1) return rc;
  const void* parts[32];
  for (int i = 0; i < pl.split; i++) parts[i] = wsb + (size_t)i * M * N * sizeof(uint16_t);
  return combine(parts, pl.split);
}

// ------------------------------------------------------------------------------------------------
// One-launch compositions for decode-sized batches: the producer of a GEMM's activations runs inside the GEMM while
// it stages them.  Both evaluate exactly the expressions of the two-launch forms (shared device functions), so a
// caller may take either; both return TBIK_ERR_UNSUPPORTED when the one-launch kernel does not apply to the shape,
// and the caller then runs the two launches.
// ------------------------------------------------------------------------------------------------
int rmsnorm_gemm_dispatch(const void* x, int64_t ldx, const void* res, int64_t ldr, const void* norm_w, float eps,
                          void* res_out, int64_t ldro, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc,
                          int M, int N, int K, const void* bias, hipStream_t stream) {
  if (M < 0 || N < 0 || K <= 0) return TBIK_ERR_INVALID;
  if (!x || !B || !C || (res && !res_out)) return TBIK_ERR_INVALID;
  if (ldb_k != 1) return TBIK_ERR_UNSUPPORTED;  // the weight as nn.Linear stores it
  if (M == 0 || N == 0) return TBIK_ERR_UNSUPPORTED;
  if (ldx < K || ldb_n < K || ldc < N || (res && (ldr < K || ldro < K))) return TBIK_ERR_INVALID;
  auto bad = [](const void* p, int64_t ld) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0 || (ld & 7) != 0; };
  if (bad(x, ldx) || bad(B, ldb_n) || (K & 7) || (res && (bad(res, ldr) || bad(res_out, ldro))) || (norm_w && bad(norm_w, 8)))
    return TBIK_ERR_ALIGNMENT;
  if (reinterpret_cast<uintptr_t>(C) & 1) return TBIK_ERR_ALIGNMENT;
  // every work-group reads x and the residual while the first one stores the new residual
  if (res_out && (res_out == x || res_out == res)) return TBIK_ERR_INVALID;
  const int vec_store = ((reinterpret_cast<uintptr_t>(C) & 7) == 0 && (ldc & 3) == 0) ? 1 : 0;
  StreamArgs sa{static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(B), static_cast<uint16_t*>(C),
                static_cast<const uint16_t*>(bias), ldx, ldb_n, ldc, M, N, K, vec_store};
  StreamNormArgs na;
  na.res = static_cast<const uint16_t*>(res);
  na.w = static_cast<const uint16_t*>(norm_w);
  na.res_out = static_cast<uint16_t*>(res_out);
  na.ldr = ldr;
  na.ldro = ldro;
  na.eps = eps;
  return gemm_single_acc_stream_norm_launch(sa, na, stream);
}

int gemm_tree_gated_dispatch(const void* gate, const void* up, int64_t ld, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                             int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, hipStream_t stream) {
  if (M < 0 || N < 0 || K <= 0) return TBIK_ERR_INVALID;
  if (!gate || !up || !B || !C) return TBIK_ERR_INVALID;
  if (leaf_k != 256 && leaf_k != 128) return TBIK_ERR_UNSUPPORTED;
  if (ldb_k != 1 || M == 0 || N == 0) return TBIK_ERR_UNSUPPORTED;
  if (ld < K || ldb_n < K || ldc < N) return TBIK_ERR_INVALID;
  if (!aligned16(gate) || !aligned16(up) || !aligned16(B) || (ld & 7) || (ldb_n & 7) || (K & 7)) return TBIK_ERR_ALIGNMENT;
  if (reinterpret_cast<uintptr_t>(C) & 1) return TBIK_ERR_ALIGNMENT;
  int T, flb, level_k;
  if (tbik_tree_params(K, leaf_k, &T, &flb, &level_k) != TBIK_OK) return TBIK_ERR_INVALID;
  const int waves = gemm_tree_strip_gated_waves(M, N, K, level_k - 1);
  if (!waves) return TBIK_ERR_UNSUPPORTED;
  const int vec_store = ((reinterpret_cast<uintptr_t>(C) & 7) == 0 && (ldc & 3) == 0) ? 1 : 0;
  StripArgs sa{static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(B), static_cast<uint16_t*>(C),
               static_cast<const uint16_t*>(bias), ld, ldb_n, ldc, M, N, K, flb, level_k - 1, vec_store,
               static_cast<const uint16_t*>(up)};
  return gemm_tree_strip_gated_launch(sa, leaf_k, waves, stream);
}

// The merged gate/up projection with the activation behind it in the same launch: out[M, inter] = silu(x Wg^T) * (x Wu^T),
// W = [2*inter, K] (rows 0 .. inter-1 gate, the rest up; the nn.Linear layout), both products rounded to bf16 first.
// TBIK_ERR_UNSUPPORTED (nothing launched) outside the row counts of the windowed streaming kernel.
int gemm_silu_mul_dispatch(const void* x, int64_t ldx, const void* W, int64_t ldw, void* out, int64_t ldo, int M, int inter, int K,
                           hipStream_t stream) {
  if (M < 0 || inter <= 0 || K <= 0) return TBIK_ERR_INVALID;
  if (M == 0) return TBIK_ERR_UNSUPPORTED;
  if (!x || !W || !out) return TBIK_ERR_INVALID;
  if (ldx < K || ldw < K || ldo < inter) return TBIK_ERR_INVALID;
  if (!aligned16(x) || !aligned16(W) || (ldx & 7) || (ldw & 7) || (K & 7)) return TBIK_ERR_ALIGNMENT;
  if (reinterpret_cast<uintptr_t>(out) & 1) return TBIK_ERR_ALIGNMENT;
  StreamArgs sa{static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(W), static_cast<uint16_t*>(out), nullptr, ldx, ldw, ldo,
                M, inter, K, ((reinterpret_cast<uintptr_t>(out) & 7) == 0 && (ldo & 3) == 0) ? 1 : 0,
                static_cast<const uint16_t*>(W) + (int64_t)inter * ldw};
  return gemm_single_acc_stream_gated_launch(sa, stream);
}

}  // namespace tbik
