// Tree-ordered 16-bit GEMM for gfx950, decode-sized M (at most 16 rows): one launch, no workspace.
//
// With a handful of rows the call is one pass over the weight matrix and the only question is how many bytes are
// in flight.  A work-group owns ONE strip of 16 weight rows (16 output columns) and cuts K over its S waves into
// S aligned subtrees of the merge tree; every wave streams its part of the strip straight from global memory
// into MFMA fragments (a lane's 16 bytes ARE its fragment: row lane%16, k = 8*(lane/16)..+7 of the 32-wide
// step), three chunks of four steps in rotation, runs the leaves of its subtree in order (level 0 left to right
// over FLB leaves, adjacent pairs above, every node rounded to the element type) and leaves the subtree's value
// in LDS; the first wave then adds the S values in the same adjacent-pair order, which is the rest of the tree.
// The arithmetic per element -- MFMA chain per leaf, k ascending, and the tree -- is that of gemm_tiled.hip and
// gemm_tree_wide.hip, hence the same bits; what differs is that the shard partials never leave the CU.
// Replaces matmul_kernel_tp_persistent, src/tbik/tree_based_matmul.py:50-187, for a few rows (the kernel itself takes up to 16).
#include "common.h"
#include "gemm_args.h"
#include "silu_mul.h"

namespace tbik {

namespace strip {
constexpr int U = 4;         // 32-wide k steps per register chunk (128 k)
constexpr int MAXLEV = 3;    // binary levels a wave keeps for its own groups (at most 8 groups per wave)
}  // namespace strip

// CPL: chunks per leaf (2 = leaf 256, 1 = leaf 128); S: waves per work-group = subtrees K is cut into.
// GATED: p.X and p.X2 are the gate and the up half of the merged projection and the activations are silu(gate) * up, formed by the
// work-group once while the first weight chunks are in flight (the function of the stand-alone kernel, so the bits it
// would have written to memory) and kept in LDS, M rows of 2K + 16 bytes, from where every wave takes its fragments;
// the tree and the MFMA chains do not change, so the product is the one of the two-launch composition.
template <int CPL, int S, bool F16, bool GATED = false>
__global__ __launch_bounds__(64 * S) __attribute__((amdgpu_waves_per_eu(4, 8))) void gemm_tree_strip_kernel(const StripArgs p) {
  using namespace strip;
  using Num = Num16<F16>;
  __shared__ uint2 part[S][64];
  extern __shared__ __attribute__((aligned(16))) uint8_t act[];   // GATED only

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n0 = xcd_contiguous_tile(blockIdx.x, gridDim.x) * 16;  // every XCD streams a contiguous range of weight rows
  const int r = lane & 15, g = lane >> 4;
  const int groups = (1 << p.lb) / S;   // groups of FLB leaves in this wave's subtree (a power of two)
  const int nch = groups * p.flb * CPL;  // chunks of this wave
  const int64_t k0 = (int64_t)wave * nch * (U * 32);
  const uint16_t* wp = p.W + (int64_t)min(n0 + r, p.N - 1) * p.ldw + k0 + 8 * g;
  const uint16_t* xp = p.X + (int64_t)min(r, p.M - 1) * p.ldx + k0 + 8 * g;

  bf16x8 w0[U], w1[U], w2[U], x0[U], x1[U], x2[U];
  // chunks past the end re-read the last one and are never used: issuing every load unconditionally keeps the
  // number of loads in flight static, so the waits leave the newer chunks in flight
  auto load = [&](bf16x8* w, bf16x8* x, int c) __attribute__((always_inline)) {
    const int cc = min(c, nch - 1);
#pragma unroll
    for (int u = 0; u < U; u++) {
      w[u] = *reinterpret_cast<const bf16x8*>(wp + (int64_t)(cc * U + u) * 32);
      if constexpr (!GATED) x[u] = *reinterpret_cast<const bf16x8*>(xp + (int64_t)(cc * U + u) * 32);
    }
  };
  const int act_rowb = p.K * 2 + 16;
  const uint8_t* act_frag = act + min(r, p.M - 1) * act_rowb + (k0 + 8 * g) * 2;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  uint32_t t[2] = {0u, 0u};        // current node, packed (n, n+1), (n+2, n+3)
  uint32_t s0[2] = {0u, 0u};       // level 0: running left-to-right sum
  uint32_t sb[MAXLEV][2];          // binary levels
#pragma unroll
  for (int l = 0; l < MAXLEV; l++) sb[l][0] = sb[l][1] = 0u;
  int c0 = 0;                      // leaves absorbed at level 0
  int gc = 0;                      // groups completed (binary counter)
  int lbw = 0;                     // binary levels inside this wave's subtree
  while ((1 << lbw) < groups) lbw++;

  // One step of the merge, written without branches (every condition is uniform over the wave and becomes a
  // select): a branch around the adds would make the compiler drain the whole load queue at the join.  `fire` is
  // false for the chunks that do not end a leaf and for the padding chunks after the last one.
  auto leaf_done = [&](bool fire) __attribute__((always_inline)) {
    uint32_t u0 = Num::pack(acc[0], acc[1]), u1 = Num::pack(acc[2], acc[3]);
    const uint32_t a0 = Num::add(s0[0], u0), a1 = Num::add(s0[1], u1);
    u0 = c0 != 0 ? a0 : u0;  // level 0: left to right over FLB leaves
    u1 = c0 != 0 ? a1 : u1;
    const bool full = fire && c0 + 1 == p.flb;
    const bool stay = fire && !full;
    s0[0] = stay ? u0 : s0[0];
    s0[1] = stay ? u1 : s0[1];
    c0 = full ? 0 : (stay ? c0 + 1 : c0);
    bool active = full;  // a finished group climbs the binary counter until it finds a free level
#pragma unroll
    for (int l = 0; l < MAXLEV; l++) {
      const bool in = active && l < lbw;
      const bool bit = (gc >> l) & 1;
      const uint32_t m0 = Num::add(sb[l][0], u0), m1 = Num::add(sb[l][1], u1);
      sb[l][0] = (in && !bit) ? u0 : sb[l][0];
      sb[l][1] = (in && !bit) ? u1 : sb[l][1];
      u0 = (in && bit) ? m0 : u0;
      u1 = (in && bit) ? m1 : u1;
      active = in && bit;
    }
    gc += full ? 1 : 0;
    t[0] = fire ? u0 : t[0];
    t[1] = fire ? u1 : t[1];
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] = fire ? 0.f : acc[e];
  };
  // chunks past the end (the loop runs in threes) multiply the re-read last chunk into an accumulator nobody reads
  auto chunk = [&](const bf16x8* w, const bf16x8* x, int c) __attribute__((always_inline)) {
    if constexpr (GATED) {
      bf16x8 xa[U];
      const int cc = min(c, nch - 1);
#pragma unroll
      for (int u = 0; u < U; u++) xa[u] = *reinterpret_cast<const bf16x8*>(act_frag + (cc * U + u) * 64);
#pragma unroll
      for (int u = 0; u < U; u++) acc = Num::mfma(w[u], xa[u], acc);
    } else {
#pragma unroll
      for (int u = 0; u < U; u++) acc = Num::mfma(w[u], x[u], acc);
    }
    leaf_done(c < nch && (CPL == 1 || (c & 1)));
  };

  // the scheduling barriers keep the loads where they are written: left alone, the scheduler sinks them towards
  // their use to shorten live ranges, and the stream is no longer two chunks ahead
  if constexpr (GATED) {
    // A wave's loads return in the order they were issued: the first round of gate / up chunks is asked for BEFORE the
    // first weight chunks, so that the activations are formed while the weight stream fills.  The loads are issued
    // unconditionally (clamped to the last chunk), or the compiler would wait for the weights as well before the first
    // use.  Six chunks per thread and round: one round covers a row of 12288 with four waves.
    constexpr int R = 6, NT = 64 * S;
    const int kc = p.K / 8, total = p.M * kc;
    uint4 gq[R], uq[R];
    auto issue = [&](int base) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < R; i++) {
        const int q = min(base + (int)threadIdx.x + NT * i, total - 1);
        const int row = q / kc, c = q - row * kc;
        const int64_t off = (int64_t)row * p.ldx + c * 8;
        gq[i] = *reinterpret_cast<const uint4*>(p.X + off);
        uq[i] = *reinterpret_cast<const uint4*>(p.X2 + off);
      }
    };
    auto consume = [&](int base) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < R; i++) {
        const int q = base + (int)threadIdx.x + NT * i;
        if (q < total) {
          const int row = q / kc, c = q - row * kc;
          uint4 o;
          o.x = silu_mul_pair<F16>(gq[i].x, uq[i].x);
          o.y = silu_mul_pair<F16>(gq[i].y, uq[i].y);
          o.z = silu_mul_pair<F16>(gq[i].z, uq[i].z);
          o.w = silu_mul_pair<F16>(gq[i].w, uq[i].w);
          *reinterpret_cast<uint4*>(act + row * act_rowb + c * 16) = o;
        }
      }
    };
    issue(0);
    __builtin_amdgcn_sched_barrier(0);
    load(w0, x0, 0);
    __builtin_amdgcn_sched_barrier(0);
    load(w1, x1, 1);
    __builtin_amdgcn_sched_barrier(0);
    consume(0);
    for (int base = R * NT; base < total; base += R * NT) {
      issue(base);
      consume(base);
    }
    __syncthreads();
  } else {
    load(w0, x0, 0);
    __builtin_amdgcn_sched_barrier(0);
    load(w1, x1, 1);
  }
  for (int c = 0; c < nch; c += 3) {
    __builtin_amdgcn_sched_barrier(0);
    load(w2, x2, c + 2);
    __builtin_amdgcn_sched_barrier(0);
    chunk(w0, x0, c);
    __builtin_amdgcn_sched_barrier(0);
    load(w0, x0, c + 3);
    __builtin_amdgcn_sched_barrier(0);
    chunk(w1, x1, c + 1);
    __builtin_amdgcn_sched_barrier(0);
    load(w1, x1, c + 4);
    __builtin_amdgcn_sched_barrier(0);
    chunk(w2, x2, c + 2);
  }
  // after the last group every level has been merged: t is the value of this wave's subtree

  part[wave][lane] = make_uint2(t[0], t[1]);
  __syncthreads();
  if (wave != 0) return;
  uint32_t lo[S], hi[S];
#pragma unroll
  for (int w = 0; w < S; w++) {
    const uint2 v = part[w][lane];
    lo[w] = v.x;
    hi[w] = v.y;
  }
#pragma unroll
  for (int step = 1; step < S; step <<= 1)
#pragma unroll
    for (int left = 0; left < S; left += 2 * step) {
      lo[left] = Num::add(lo[left], lo[left + step]);
      hi[left] = Num::add(hi[left], hi[left + step]);
    }
  // lane (r, g) holds C[r][n0 + 4g .. 4g+3]; the bias joins as one more node after the tree
  const int n = n0 + 4 * g;
  if (r >= p.M || n >= p.N) return;
  uint32_t olo = lo[0], ohi = hi[0];
  if (p.bias) {
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (n + e < p.N) bv[e] = Num::to_f32(p.bias[n + e]);
    olo = Num::add(olo, Num::pack(bv[0], bv[1]));
    ohi = Num::add(ohi, Num::pack(bv[2], bv[3]));
  }
  uint16_t* dst = p.C + (int64_t)r * p.ldc + n;
  if (p.vec_store && n + 3 < p.N) {
    *reinterpret_cast<uint2*>(dst) = make_uint2(olo, ohi);
  } else {
    const uint16_t v[4] = {(uint16_t)(olo & 0xffff), (uint16_t)(olo >> 16), (uint16_t)(ohi & 0xffff), (uint16_t)(ohi >> 16)};
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (n + e < p.N) dst[e] = v[e];
  }
}

// Waves per strip for a problem, or 0 when this kernel is not the one to use.  Measured on MI355X: HBM bandwidth
// is shared about equally among the CUs that ask for it, so in a single pass over the weights the CU with the most
// strips finishes last and every CU has to carry the same number -- a grid of 320 strips (two on every fourth CU)
// streams at 3 TB/s where 256 or 512 strips reach 5 -- and the activation rows, which every lane fetches for
// itself, cost as much as the weights once there are more than a few of them (unless the tree has so few aligned subtrees that the K-cut grid of the tiled kernel
// cannot fill the chip either).  Four waves per strip are the best cut of K (two chunks of 4 KiB in flight each);
// beyond a few hundred MB of weights the tiled kernel streams as fast and nothing is gained.
int gemm_tree_strip_waves(int M, int N, int K, int lb) {
  if (lb < 1 || lb > 6 || M > 16 || (M > 4 && lb > 2)) return 0;
  if ((int64_t)N * K > 150000000) return 0;
  const int64_t strips = ((int64_t)N + 15) / 16;
  if (strips < 64) return 0;
  // half the chip or less, and a long K: the K-cut grid of the tiled kernel spreads the same weights over all CUs
  // ([1,8192] x [8192,1024] 13.1 us here, 9.4 there; [4,25600] x [25600,2048] 38.8 against 31.8; up to K = 3072 this
  // kernel is still ahead, 6.5 against 7.5 at N = 2048)
  if (strips <= 128 && K >= 4096) return 0;
  const int64_t rounds = (strips + 255) / 256;
  if (strips > 256 && rounds * 256 * 100 > strips * 115) return 0;
  if (lb == 1) return 2;
  return lb - 2 > strip::MAXLEV ? 8 : 4;
}

template <int CPL, bool F16>
static int launch_strip(const StripArgs& a, int s, hipStream_t stream) {
  const unsigned strips = (unsigned)((a.N + 15) / 16);
  switch (s) {
    case 2: hipLaunchKernelGGL((gemm_tree_strip_kernel<CPL, 2, F16>), dim3(strips), dim3(128), 0, stream, a); break;
    case 4: hipLaunchKernelGGL((gemm_tree_strip_kernel<CPL, 4, F16>), dim3(strips), dim3(256), 0, stream, a); break;
    case 8: hipLaunchKernelGGL((gemm_tree_strip_kernel<CPL, 8, F16>), dim3(strips), dim3(512), 0, stream, a); break;
    default: return TBIK_ERR_INVALID;
  }
  return hip_code(hipGetLastError());
}

template <int CPL, int S>
static int launch_strip_gated_s(const StripArgs& a, hipStream_t stream) {
  const unsigned strips = (unsigned)((a.N + 15) / 16);
  const int smem = a.M * (a.K * 2 + 16);
  auto kern = gemm_tree_strip_kernel<CPL, S, false, true>;
  if (smem > 32 * 1024) {
    static std::atomic<uint64_t> done{0};
    hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, done);
    if (e != hipSuccess) return hip_code(e);
  }
  hipLaunchKernelGGL(kern, dim3(strips), dim3(64 * S), smem, stream, a);
  return hip_code(hipGetLastError());
}

// Tree matmul of silu(gate) * up for a.X = gate, a.X2 = up ([M,K] each, row stride a.ldx), bf16: where the one-launch
// kernel applies, the activations (M rows of 2K + 16 bytes) fit the LDS and forming them in every work-group is cheaper
// than a launch of its own; 0 otherwise.  Every work-group evaluates all M * K activations, so the price grows with
// M * K and with the number of work-groups: measured on MI355X against silu_mul + tree matmul with the launches back to
// back (replays of a recorded graph, cold weights), N = 4096 (one work-group per CU), K = 12288: 21.5 / 25.3 / 28.2 us
// for 1 .. 3 rows against 22.6 / 24.3 / 24.9; K = 3072: 15 us against 26 for 1 .. 4 rows; N = 5120 (320 work-groups),
// K = 12800: 52 - 53 us against 47.5 at any row count.  Hence at most 16384 activations per work-group.
int gemm_tree_strip_gated_waves(int M, int N, int K, int lb) {
  if (M > 4 || (int64_t)M * (K * 2 + 16) > 128 * 1024) return 0;
  if ((int64_t)M * K > 16384 || (N + 15) / 16 > 256) return 0;
  return gemm_tree_strip_waves(M, N, K, lb);
}

int gemm_tree_strip_gated_launch(const StripArgs& a, int leaf_k, int waves, hipStream_t stream) {
  if (a.M <= 0 || a.M > 4 || a.N <= 0 || !a.X2 || (leaf_k != 256 && leaf_k != 128)) return TBIK_ERR_INVALID;
  if (a.flb <= 0 || a.lb < 0 || (int64_t)a.flb * leaf_k * (1 << a.lb) != a.K) return TBIK_ERR_INVALID;
  if (waves < 2 || waves > 8 || (waves & (waves - 1)) || waves > (1 << a.lb)) return TBIK_ERR_INVALID;
  if (leaf_k == 256) {
    if (waves == 2) return launch_strip_gated_s<2, 2>(a, stream);
    if (waves == 4) return launch_strip_gated_s<2, 4>(a, stream);
    return launch_strip_gated_s<2, 8>(a, stream);
  }
  if (waves == 2) return launch_strip_gated_s<1, 2>(a, stream);
  if (waves == 4) return launch_strip_gated_s<1, 4>(a, stream);
  return launch_strip_gated_s<1, 8>(a, stream);
}

int gemm_tree_strip_launch(const StripArgs& a, int leaf_k, int waves, bool f16, hipStream_t stream) {
  if (a.M <= 0 || a.M > 16 || a.N <= 0 || (leaf_k != 256 && leaf_k != 128)) return TBIK_ERR_INVALID;
  if (a.flb <= 0 || a.lb < 0 || (int64_t)a.flb * leaf_k * (1 << a.lb) != a.K) return TBIK_ERR_INVALID;
  if (waves < 2 || waves > 8 || (waves & (waves - 1)) || waves > (1 << a.lb)) return TBIK_ERR_INVALID;
  if (leaf_k == 256) return f16 ? launch_strip<2, true>(a, waves, stream) : launch_strip<2, false>(a, waves, stream);
  return f16 ? launch_strip<1, true>(a, waves, stream) : launch_strip<1, false>(a, waves, stream);
}

}  // namespace tbik
