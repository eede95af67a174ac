// Single-accumulator 16-bit GEMM for gfx950, decode-sized M (at most 64 rows): the batch-invariant aten::mm /
// aten::addmm of the reference (matmul_persistent, src/bio/batch_invariant_ops.py:127-197) when the batch is a
// handful of tokens and the call is one pass over the weight matrix.
//
// The accumulation contract of the batch-invariant mm forbids a split over K (one fp32 accumulator per element,
// k ascending), so the only parallelism is over N.  Every wave therefore owns ONE strip of 16 weight rows (16
// output columns, all M rows) and streams it straight from global memory into MFMA fragments -- a lane's 16
// bytes ARE its fragment: row lane%16, k = 8*(lane/16)..+7 of the 32-wide step -- a whole window of 16 or 32
// steps ahead, so that a few hundred independent waves keep enough bytes in flight to load the memory system.  The
// activations are small and shared: the waves of a work-group (2 or 4 strips) stage each window of X in LDS once
// (double-buffered, one barrier per window), which keeps the vector-memory queue of every wave for the weights.
// With a handful of rows all of X is staged up front and the waves never meet again; work-groups shrink to one
// or two strips when N is small, so that every CU gets some.  Same MFMA chain per element as the tiled and the
// quad kernels, hence the same bits.
#include "common.h"
#include "gemm_args.h"
#include "rmsnorm_row.h"
#include "silu_mul.h"

namespace tbik {

namespace stream {
// LDS bytes per X row of a window of `ws` steps: 16 bytes of padding spread the 16 rows of a fragment read over all banks
constexpr int rowb(int ws) { return ws * 64 + 16; }
}  // namespace stream

// Epilogue shared by the two kernels: lane (m = r, g) holds C[16 b + r][n0 + 4g .. 4g+3]; the bias joins in fp32
// before the single rounding.
template <int MB, bool F16>
__device__ __forceinline__ void stream_store(const StreamArgs& p, const f32x4* acc, int n0, int r, int g) {
  using Num = Num16<F16>;
  const int n = n0 + 4 * g;
  if (n >= p.N) return;
  float bv[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.bias) {
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (n + e < p.N) bv[e] = Num::to_f32(p.bias[n + e]);
  }
#pragma unroll
  for (int b = 0; b < MB; b++) {
    const int m = b * 16 + r;
    if (m >= p.M) continue;
    const uint32_t lo = Num::pack(acc[b][0] + bv[0], acc[b][1] + bv[1]);
    const uint32_t hi = Num::pack(acc[b][2] + bv[2], acc[b][3] + bv[3]);
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

// Gated epilogue: gate and up are rounded to the element type exactly as stream_store rounds them (no bias), then
// silu(gate) * up as the stand-alone activation kernel computes it (silu_mul.h).
template <int MB, bool F16>
__device__ __forceinline__ void stream_store_gated(const StreamArgs& p, const f32x4* gate, const f32x4* up, int n0, int r, int g) {
  using Num = Num16<F16>;
  const int n = n0 + 4 * g;
  if (n >= p.N) return;
  const float z = 0.f;  // the plain epilogue adds a zero bias in fp32: an accumulator of -0 becomes +0 there, so here too
#pragma unroll
  for (int b = 0; b < MB; b++) {
    const int m = b * 16 + r;
    if (m >= p.M) continue;
    const uint32_t glo = Num::pack(gate[b][0] + z, gate[b][1] + z), ghi = Num::pack(gate[b][2] + z, gate[b][3] + z);
    const uint32_t ulo = Num::pack(up[b][0] + z, up[b][1] + z), uhi = Num::pack(up[b][2] + z, up[b][3] + z);
    const uint32_t lo = silu_mul_pair<F16>(glo, ulo), hi = silu_mul_pair<F16>(ghi, uhi);
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

// A few rows (M * K small enough for LDS): all of X is staged once, one barrier, and then every wave runs on its
// own -- nothing couples a wave's stream of weight loads to its neighbours'.
//
// NORM > 0: the activations are RMSNorm(x [+ residual]) * weight, computed by the work-group while it stages them -- one
// wavefront per row with the row function of the stand-alone RMSNorm kernel (NORM = its chunks per lane: 8 for rows
// of up to 4096 elements, 16 up to 8192), so the staged values are the bits that kernel would have written to memory,
// and the product is the one of the two-launch composition.  Every work-group normalises all M rows for itself (a few
// KB from the L2); the first one also stores the new residual.  The norm's loads follow the first weight loads into
// the memory queue, so its latency is covered by the start of the weight stream.
constexpr int ROWS_U = 16;        // steps per register chunk (two chunks in flight)
constexpr int ROWS_MAX_ELEMS = 32768;  // M * K at most: two rounds of staging loads in a work-group of 4 waves
template <int NWAVES, bool F16, int NORM = 0>   // strips per work-group: 1 when N is small, so that every CU gets some
__global__ __launch_bounds__(NWAVES * 64) void gemm_single_acc_stream_rows_kernel(const StreamArgs p, const StreamNormArgs nrm) {
  using Num = Num16<F16>;
  constexpr int NW = NWAVES, NT = NWAVES * 64;
  constexpr int U = ROWS_U;
  extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // M rows of 2K + 16 bytes

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // every XCD streams a contiguous range of the weight rows (lm_head at 8 rows: 228 -> 211 us)
  const int n0 = (xcd_contiguous_tile(blockIdx.x, gridDim.x) * NW + wave) * 16;
  const int r = lane & 15, g = lane >> 4;
  const uint16_t* wp = p.W + (int64_t)min(n0 + r, p.N - 1) * p.ldw + 8 * g;
  const int nsteps = p.K / 32;
  const int nchunks = nsteps / U;
  const int rowb = p.K * 2 + 16;

  bf16x8 wa[U], wb[U];
  auto load = [&](bf16x8* w, int c) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; u++) w[u] = *reinterpret_cast<const bf16x8*>(wp + (int64_t)(c * U + u) * 32);
  };
  if constexpr (NORM > 0) {
    // A wave's loads return in the order they were issued: the row this wave normalises is asked for FIRST, then the
    // first chunk of weights, so that the norm (loads, a reduction over the wave, LDS) runs while the weight stream
    // fills.  No load sits under a branch (a wave without a row of its own loads the last row and drops it; the
    // launcher guarantees a whole chunk of weights), or the compiler would wait for the weights before the norm.
    RmsnormRow<NORM, F16, true> row;
    const bool mine = wave < p.M;
    const int myrow = min(wave, p.M - 1);
    row.load(p.X + (int64_t)myrow * p.ldx, nrm.res ? nrm.res + (int64_t)myrow * nrm.ldr : nullptr, nrm.w, p.K, lane);
    __builtin_amdgcn_sched_barrier(0);   // the scheduler would put the weight loads first
    load(wa, 0);
    __builtin_amdgcn_sched_barrier(0);
    if (mine) {
      uint8_t* dst = xs + wave * rowb;
      row.finish((nrm.res_out && blockIdx.x == 0) ? nrm.res_out + (int64_t)wave * nrm.ldro : nullptr, p.K, nrm.eps, lane,
                 [&](int c, const uint4& o) { *reinterpret_cast<uint4*>(dst + c * 16) = o; });
    }
    for (int m = wave + NW; m < p.M; m += NW) {   // more rows than waves: the others queue behind the weights
      uint8_t* dst = xs + m * rowb;
      rmsnorm_row<NORM, F16>(p.X + (int64_t)m * p.ldx, nrm.res ? nrm.res + (int64_t)m * nrm.ldr : nullptr, nrm.w,
                             (nrm.res_out && blockIdx.x == 0) ? nrm.res_out + (int64_t)m * nrm.ldro : nullptr, p.K, nrm.eps,
                             lane, [&](int c, const uint4& o) { *reinterpret_cast<uint4*>(dst + c * 16) = o; });
    }
  } else {
    if (nchunks > 0) load(wa, 0);  // the weights start flowing before X is staged
    const int kc = p.K / 8, total = p.M * kc;
    for (int base = 0; base < total; base += NT * 8) {  // one or two rounds of 8 loads in flight per thread
      u32x4 xr[8];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int q = base + tid + NT * i;
        if (q < total) xr[i] = *reinterpret_cast<const u32x4*>(p.X + (int64_t)(q / kc) * p.ldx + (q % kc) * 8);
      }
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int q = base + tid + NT * i;
        if (q < total) *reinterpret_cast<u32x4*>(xs + (q / kc) * rowb + (q % kc) * 16) = xr[i];
      }
    }
  }
  __syncthreads();

  f32x4 acc[1] = {f32x4{0.f, 0.f, 0.f, 0.f}};
  const uint8_t* xrow = xs + min(r, p.M - 1) * rowb + g * 16;
  auto mma = [&](const bf16x8* w, int c) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const bf16x8 x = *reinterpret_cast<const bf16x8*>(xrow + (c * U + u) * 64);
      acc[0] = Num::mfma(w[u], x, acc[0]);
    }
  };
  int c = 0;
  for (; c + 2 <= nchunks; c += 2) {
    load(wb, c + 1);
    mma(wa, c);
    if (c + 2 < nchunks) load(wa, c + 2);
    mma(wb, c + 1);
  }
  if (c < nchunks) mma(wa, c);  // odd number of chunks: the last one is already in registers
  for (int s = nchunks * U; s < nsteps; s++) {
    const bf16x8 w = *reinterpret_cast<const bf16x8*>(wp + (int64_t)s * 32);
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(xrow + s * 64);
    acc[0] = Num::mfma(w, x, acc[0]);
  }
  stream_store<1, F16>(p, acc, n0, r, g);
}

// GATED: a wave owns strip n0 of BOTH weight matrices (gate and up of a merged projection) and runs the pass over K twice,
// once per matrix (X is staged again: it comes from the L2), then stores silu(gate) * up: the consumer of the two products
// inside their producer, one launch and a third of the output bytes.
template <int MB, int WS, int NWAVES, bool F16, bool GATED = false>  // MB blocks of 16 activation rows, windows of WS steps (32 k each)
__global__ __launch_bounds__(NWAVES * 64) void gemm_single_acc_stream_kernel(const StreamArgs p) {
  using namespace stream;
  using Num = Num16<F16>;
  constexpr int NW = NWAVES, NT = NWAVES * 64;
  constexpr int KW = WS * 32;
  constexpr int ROWB = rowb(WS);
  constexpr int ROWS = MB * 16;
  constexpr int XBUF = ROWS * ROWB;
  constexpr int XCHUNKS = ROWS * (KW / 8);          // 16-byte chunks of a window of X
  constexpr int XLD = (XCHUNKS + NT - 1) / NT;      // loads per thread per window; where NT does not divide the chunks,
                                                    // the threads past the end move the last chunk once more
  extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // two X windows of XBUF bytes

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // every XCD streams a contiguous range of the weight rows (lm_head at 8 rows: 228 -> 211 us)
  const int n0 = (xcd_contiguous_tile(blockIdx.x, gridDim.x) * NW + wave) * 16;
  const int r = lane & 15, g = lane >> 4;

  const uint16_t* wp = p.W + (int64_t)min(n0 + r, p.N - 1) * p.ldw + 8 * g;  // (the second pass of the gated form moves it)

  // staging of X: thread t moves 16-byte chunk q % (KW/8) of row q / (KW/8), q = t + NT i, i < XLD
  const uint16_t* xsrc[XLD];
  uint32_t xdst[XLD];
#pragma unroll
  for (int i = 0; i < XLD; i++) {
    const int q = min(tid + NT * i, XCHUNKS - 1);
    const int row = q / (KW / 8), c = q % (KW / 8);
    xsrc[i] = p.X + (int64_t)min(row, p.M - 1) * p.ldx + c * 8;
    xdst[i] = row * ROWB + c * 16;
  }
  const int nsteps = p.K / 32;
  const int nfull = nsteps / WS;  // whole windows; the steps after them are handled at the end

  u32x4 xr[XLD];
  bf16x8 wa[WS], wb[WS];
  // Every load of the main loop is issued unconditionally and addresses a whole window (one base pointer, constant
  // offsets): a window past the end re-reads the last one and is never used, so the number of loads in flight is
  // static and the waits can leave the next window in flight.
  auto load_x = [&](int w) __attribute__((always_inline)) {
    const int64_t off = (int64_t)min(w, nfull - 1) * KW;
#pragma unroll
    for (int i = 0; i < XLD; i++) xr[i] = *reinterpret_cast<const u32x4*>(xsrc[i] + off);
  };
  auto store_x = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < XLD; i++) *reinterpret_cast<u32x4*>(xs + buf * XBUF + xdst[i]) = xr[i];
  };
  auto load_w = [&](bf16x8* w, int win) __attribute__((always_inline)) {
    const uint16_t* base = wp + (int64_t)min(win, nfull - 1) * KW;
#pragma unroll
    for (int u = 0; u < WS; u++) w[u] = *reinterpret_cast<const bf16x8*>(base + u * 32);
  };

  f32x4 acc[MB];
#pragma unroll
  for (int b = 0; b < MB; b++) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
  const uint32_t xfrag = r * ROWB + g * 16;
  auto compute = [&](const bf16x8* w, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < WS; u++) {
#pragma unroll
      for (int b = 0; b < MB; b++) {
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(xs + buf * XBUF + xfrag + b * 16 * ROWB + u * 64);
        acc[b] = Num::mfma(w[u], x, acc[b]);
      }
    }
  };

  auto pass = [&]() __attribute__((always_inline)) {
  if (nfull > 0) {
    load_x(0);
    load_w(wa, 0);
    store_x(0);
    __syncthreads();
    int win = 0;
    for (; win + 1 < nfull; win += 2) {
      // even window: weights in wa, X in buffer 0
      __builtin_amdgcn_sched_barrier(0);
      load_x(win + 1);
      load_w(wb, win + 1);
      __builtin_amdgcn_sched_barrier(0);
      compute(wa, 0);
      store_x(1);
      __syncthreads();
      // odd window: weights in wb, X in buffer 1
      __builtin_amdgcn_sched_barrier(0);
      load_x(win + 2);
      load_w(wa, win + 2);
      __builtin_amdgcn_sched_barrier(0);
      compute(wb, 1);
      store_x(0);
      __syncthreads();
    }
    if (win < nfull) compute(wa, 0);  // an odd number of windows: the last one is already in wa and buffer 0
  }
  // the steps after the last whole window (K not a multiple of the window): fragments straight from global memory
  for (int s = nfull * WS; s < nsteps; s++) {
    const bf16x8 w = *reinterpret_cast<const bf16x8*>(wp + (int64_t)s * 32);
#pragma unroll
    for (int b = 0; b < MB; b++) {
      const bf16x8 x = *reinterpret_cast<const bf16x8*>(p.X + (int64_t)min(b * 16 + r, p.M - 1) * p.ldx + (int64_t)s * 32 + 8 * g);
      acc[b] = Num::mfma(w, x, acc[b]);
    }
  }
  };
  pass();
  if constexpr (GATED) {
    f32x4 gate[MB];
#pragma unroll
    for (int b = 0; b < MB; b++) {
      gate[b] = acc[b];
      acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();  // every wave is through with the last window of X before it is staged again
    wp = p.W2 + (int64_t)min(n0 + r, p.N - 1) * p.ldw + 8 * g;
    pass();
    stream_store_gated<MB, F16>(p, gate, acc, n0, r, g);
  } else {
    stream_store<MB, F16>(p, acc, n0, r, g);
  }
}

template <int MB, int WS, int NWAVES, bool F16, bool GATED = false>
static int stream_launch_nw(const StreamArgs& a, hipStream_t stream) {
  const int64_t groups = ((int64_t)a.N + 16 * NWAVES - 1) / (16 * NWAVES);
  if (groups > 0x7fffffff) return TBIK_ERR_INVALID;
  constexpr int smem = 2 * MB * 16 * stream::rowb(WS);
  auto kern = gemm_single_acc_stream_kernel<MB, WS, NWAVES, F16, GATED>;
  if (smem > 64 * 1024) {
    static std::atomic<uint64_t> done{0};
    hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, done);
    if (e != hipSuccess) return hip_code(e);
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)groups), dim3(NWAVES * 64), smem, stream, a);
  return hip_code(hipGetLastError());
}

template <int MB, int WS, bool F16, bool GATED = false>
static int stream_launch(const StreamArgs& a, hipStream_t stream) {
  // Strips per work-group.  More strips share each staged window of X (gate_up of an 8B model at M=64: 80 us with four
  // strips per work-group, 55 us with eight), but HBM bandwidth is shared about equally among the CUs that ask for it,
  // so the CU with the most work-groups finishes last.  The estimate is the pass over the weights, stretched by the share
  // of CU slots that the last round of work-groups leaves idle, plus the restaging of X per strip at a third of the
  // price of a weight byte (it comes from the L2).  Measured: gate_up at M=32 (1536 strips) 48.4 us as 384 groups of
  // four (two on every second CU), 41.2 us as 256 groups of six; [32,4096]x[4096,18432] 48.6 -> 35.4; lm_head (9496
  // strips, ten rounds of groups of four) is within 2 % for three, four and six.
  const int64_t strips = ((int64_t)a.N + 15) / 16;
  // grids of many rounds do not run in rounds: the last one matters little there, the restaging of X more
  if (strips > 4 * 1024) return MB >= 3 ? stream_launch_nw<MB, WS, 8, F16, GATED>(a, stream) : stream_launch_nw<MB, WS, 4, F16, GATED>(a, stream);
  static const int cand[5] = {8, 6, 4, 3, 2};
  int best = 4;
  double best_cost = 0.0;
  for (int i = 0; i < 5; i++) {
    const int nw = cand[i];
    if (nw == 8 && (MB < 3 || strips < 1536)) continue;  // eight strips per group: many rows and a large grid only
    if (nw == 2 && MB > 2) continue;                     // two: one or two blocks of rows only
    const int64_t groups = (strips + nw - 1) / nw;
    const double fill = (double)groups / (double)(((groups + 255) / 256) * 256);
    const double cost = (1.0 + 0.35 * (double)a.M / (16.0 * nw)) / fill;
    if (best_cost == 0.0 || cost < best_cost) {
      best_cost = cost;
      best = nw;
    }
  }
  switch (best) {
    case 8: return stream_launch_nw<MB, WS, 8, F16, GATED>(a, stream);
    case 6: return stream_launch_nw<MB, WS, 6, F16, GATED>(a, stream);
    case 3: return stream_launch_nw<MB, WS, 3, F16, GATED>(a, stream);
    case 2: return stream_launch_nw<MB, WS, (MB <= 2 ? 2 : 4), F16, GATED>(a, stream);
    default: return stream_launch_nw<MB, WS, 4, F16, GATED>(a, stream);
  }
}

template <int NWAVES, bool F16, int NORM = 0>
static int stream_rows_launch(const StreamArgs& a, hipStream_t stream, const StreamNormArgs& nrm = StreamNormArgs{}) {
  const int64_t groups = ((int64_t)a.N + 16 * NWAVES - 1) / (16 * NWAVES);
  if (groups > 0x7fffffff) return TBIK_ERR_INVALID;
  const int smem = a.M * (a.K * 2 + 16);
  hipLaunchKernelGGL((gemm_single_acc_stream_rows_kernel<NWAVES, F16, NORM>), dim3((unsigned)groups), dim3(NWAVES * 64), smem,
                     stream, a, nrm);
  return hip_code(hipGetLastError());
}

// Strips per work-group of the whole-X kernel.  HBM bandwidth is shared about equally among the CUs that ask for it, so
// the CU with the most work-groups finishes last and the grid should put the same number on every CU: the score is the
// share of CU slots that the last round of work-groups leaves used (measured: gate_up of an 8B model, 1536 strips, 41 us
// as 384 groups of four, 37 us as 512 groups of three).  One strip per work-group restages X for every strip and is only
// considered while X is small; two strips per work-group measured worse than either neighbour throughout.
static int stream_rows_waves(const StreamArgs& a) {
  const int64_t strips = ((int64_t)a.N + 15) / 16;
  auto score = [&](int nw, double weight) {
    const int64_t groups = (strips + nw - 1) / nw;
    return weight * (double)groups / (double)(((groups + 255) / 256) * 256);
  };
  const double s3 = score(3, 1.0), s4 = score(4, 0.98);
  const double s1 = a.M * a.K <= ROWS_MAX_ELEMS / 4 ? score(1, 0.95) : 0.0;
  if (s1 > s3 && s1 > s4) return 1;
  return s3 >= s4 ? 3 : 4;
}

// all of X fits the staging registers of one pass and 40 KiB of LDS (several work-groups per CU)
static bool stream_rows_applies(const StreamArgs& a) {
  return a.M <= 16 && (int64_t)a.M * a.K <= ROWS_MAX_ELEMS && (int64_t)a.M * (a.K * 2 + 16) <= 40 * 1024;
}

// mm of RMSNorm(x [+ residual]) * weight in one launch: only where the whole-X kernel applies (a few rows) and the
// row length is one the stand-alone norm kernel takes; TBIK_ERR_UNSUPPORTED otherwise (the caller runs the two launches).
int gemm_single_acc_stream_norm_launch(const StreamArgs& a, const StreamNormArgs& nrm, hipStream_t stream) {
  // K >= 512: the kernel issues its first chunk of weight loads (16 steps of 32) unconditionally
  if (a.M <= 0 || (a.K & 31) != 0 || a.K < 512 || a.K > 8192 || !stream_rows_applies(a)) return TBIK_ERR_UNSUPPORTED;
  const int nw = stream_rows_waves(a);
  if (a.K <= 4096) {
    if (nw == 1) return stream_rows_launch<1, false, 8>(a, stream, nrm);
    if (nw == 3) return stream_rows_launch<3, false, 8>(a, stream, nrm);
    return stream_rows_launch<4, false, 8>(a, stream, nrm);
  }
  if (nw == 1) return stream_rows_launch<1, false, 16>(a, stream, nrm);
  if (nw == 3) return stream_rows_launch<3, false, 16>(a, stream, nrm);
  return stream_rows_launch<4, false, 16>(a, stream, nrm);
}

// ... and is the faster of the two.  Every work-group of the whole-X kernel stages all of X before it streams, the
// windowed kernel a window at a time behind its first weights.  Measured on MI355X (cold weights, launches back to back):
// the whole-X kernel wins on wide weight matrices (gate_up, 24576 rows: 38.4 against 41.4 us at one row of 4096) and
// while X is small; it loses from a few thousand elements of X on -- [4,4096] x [4096,6144] 16.7 against 13.0 us,
// [2,8192] x [8192,5120] 29.2 against 22.8, [1,12288] x [12288,4096] 38.3 against 29.9, [8,2048] x [2048,4096] 10.1
// against 7.2 -- the earlier the more strips there are.
static bool stream_rows_pays(const StreamArgs& a) {
#ifdef TBIK_STREAM_ROWS_ALWAYS
  return true;
#endif
  const int64_t xe = (int64_t)a.M * a.K;
  if (a.K < 512) return true;   // shorter than one window: nothing to stage behind
  return a.N >= 10240 || xe <= 2048 || (xe <= 4096 && a.N <= 4096) || (xe <= 8192 && a.N <= 3072);
}

// Requires 0 < M <= 64 and K a multiple of 32 (checked by the dispatcher).
int gemm_single_acc_stream_launch(const StreamArgs& a, bool f16, hipStream_t stream) {
  if (a.M <= 0 || a.M > 64 || (a.K & 31) != 0) return TBIK_ERR_UNSUPPORTED;
  if (stream_rows_applies(a) && stream_rows_pays(a)) {
    const int nw = stream_rows_waves(a);
    if (nw == 1) return f16 ? stream_rows_launch<1, true>(a, stream) : stream_rows_launch<1, false>(a, stream);
    if (nw == 3) return f16 ? stream_rows_launch<3, true>(a, stream) : stream_rows_launch<3, false>(a, stream);
    return f16 ? stream_rows_launch<4, true>(a, stream) : stream_rows_launch<4, false>(a, stream);
  }
  const int mb = (a.M + 15) / 16;
  if (f16) {
    switch (mb) {
      case 1: return stream_launch<1, 16, true>(a, stream);
      case 2: return stream_launch<2, 16, true>(a, stream);
      case 3: return stream_launch<3, 16, true>(a, stream);
      default: return stream_launch<4, 16, true>(a, stream);
    }
  }
  switch (mb) {
    case 1: return stream_launch<1, 16, false>(a, stream);
    case 2: return stream_launch<2, 16, false>(a, stream);
    case 3: return stream_launch<3, 16, false>(a, stream);
    default: return stream_launch<4, 16, false>(a, stream);
  }
}

// The gated form: only the windowed kernel has it (5 .. 64 rows: fewer rows take the whole-X kernel, whose consumer, the
// tree matmul of down_proj, forms the activation itself).
int gemm_single_acc_stream_gated_launch(const StreamArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.M > 64 || (a.K & 31) != 0 || a.K < 32 * 16 || !a.W2 || a.bias || (a.N & 15) != 0) return TBIK_ERR_UNSUPPORTED;
  if (stream_rows_applies(a)) return TBIK_ERR_UNSUPPORTED;
  switch ((a.M + 15) / 16) {
    case 1: return stream_launch<1, 16, false, true>(a, stream);
    case 2: return stream_launch<2, 16, false, true>(a, stream);
    case 3: return stream_launch<3, 16, false, true>(a, stream);
    default: return stream_launch<4, 16, false, true>(a, stream);
  }
}

}  // namespace tbik
