// Batch-invariant row reductions for gfx950: RMSNorm (bf16 or fp16), log_softmax / softmax (fp32, bf16, fp16), mean.
//
// Rule shared by all kernels here: the decomposition of a row into lanes, wavefronts and segments,
// and the order in which partial sums meet, is a function of the ROW LENGTH only.  The number of rows
// only changes how many identical work-groups are launched.  No atomics, no split decided at run time.
#include "common.h"
#include "rmsnorm_row.h"

namespace tbik {

// ================================================================================================
// RMSNorm, one wavefront per row (4 rows per 256-thread block), the row held in registers.
// Lane l owns the 16-byte chunks l, l+64, l+128, ...; sum of squares: sequentially inside a lane,
// then the fixed butterfly across lanes.
// Arithmetic follows vLLM RMSNorm.forward_native, which the reference routes to
// (src/patch/patch_batch_invariant.py:9-16): fp32 math, normalised value rounded to bf16, then a bf16
// multiply by the weight.
// ================================================================================================
struct RmsArgs {
  const uint16_t* x;
  const uint16_t* res;
  const uint16_t* w;
  uint16_t* out;
  uint16_t* res_out;
  int64_t ldx, ldr, ldo, ldro;
  int64_t rows;
  int hidden;
  float eps;
};

template <int CPL, bool F16>  // chunks (8 elements) per lane kept in registers; bf16 or fp16 elements
__global__ __launch_bounds__(256) void rmsnorm_kernel(const RmsArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  uint4* orow = reinterpret_cast<uint4*>(a.out + row * a.ldo);
  rmsnorm_row<CPL, F16>(a.x + row * a.ldx, a.res ? a.res + row * a.ldr : nullptr, a.w,
                        a.res_out ? a.res_out + row * a.ldro : nullptr, a.hidden, a.eps, lane,
                        [&](int c, const uint4& o) { orow[c] = o; });
}

template <bool F16>
static void rmsnorm_launch(const RmsArgs& a, int cpl, dim3 grid, hipStream_t stream) {
  const dim3 block(256);
  if (cpl <= 1) hipLaunchKernelGGL((rmsnorm_kernel<1, F16>), grid, block, 0, stream, a);
  else if (cpl <= 2) hipLaunchKernelGGL((rmsnorm_kernel<2, F16>), grid, block, 0, stream, a);
  else if (cpl <= 4) hipLaunchKernelGGL((rmsnorm_kernel<4, F16>), grid, block, 0, stream, a);
  else if (cpl <= 8) hipLaunchKernelGGL((rmsnorm_kernel<8, F16>), grid, block, 0, stream, a);
  else hipLaunchKernelGGL((rmsnorm_kernel<16, F16>), grid, block, 0, stream, a);
}

int rmsnorm_dispatch(const void* x, int64_t ldx, const void* res, int64_t ldr, const void* w, void* out, int64_t ldo,
                     void* res_out, int64_t ldro, int64_t rows, int hidden, float eps, bool f16, hipStream_t stream) {
  if (rows < 0 || hidden <= 0) return TBIK_ERR_INVALID;
  if (rows == 0) return TBIK_OK;
  if (!x || !out) return TBIK_ERR_INVALID;
  if (res && !res_out) return TBIK_ERR_INVALID;
  if (rows == 0) return TBIK_OK;
  if (hidden & 7) return TBIK_ERR_ALIGNMENT;
  auto bad = [](const void* p, int64_t ld) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0 || (ld & 7) != 0; };
  if (bad(x, ldx) || bad(out, ldo) || (res && (bad(res, ldr) || bad(res_out, ldro))) || (w && bad(w, 8)))
    return TBIK_ERR_ALIGNMENT;
  if (hidden > 16 * 512) return TBIK_ERR_UNSUPPORTED;
  RmsArgs a{static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(res), static_cast<const uint16_t*>(w),
            static_cast<uint16_t*>(out), static_cast<uint16_t*>(res_out), ldx, ldr, ldo, ldro, rows, hidden, eps};
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffff) return TBIK_ERR_INVALID;
  const dim3 grid((unsigned)blocks);
  const int cpl = (hidden + 511) / 512;  // a function of the row length only
  if (f16) rmsnorm_launch<true>(a, cpl, grid, stream);
  else rmsnorm_launch<false>(a, cpl, grid, stream);
  return hip_code(hipGetLastError());
}

// ================================================================================================
// log_softmax / softmax over the last dimension; fp32, bf16 or fp16 in, the same type or fp32 out, fp32 arithmetic.
// Replaces the one-program-per-row three-pass kernel of the reference (src/bio/batch_invariant_ops.py:200-260, which
// loads the input dtype directly, :263-301).
//
// Arithmetic (a function of `cols` alone): a row is cut into fixed segments of 4096 elements.  Inside a segment,
// thread t of 256 owns the 4-element chunks t, t+256, t+512, t+768; a segment reduces to (max, sum of exp(x - max))
// by: per-thread sequential, fixed butterfly over the wavefront, four wavefronts joined in order.  The segment pairs
// of a row are merged by one wavefront (lane l takes segments l, l+64, ... ascending, then the butterfly).
//
// Two schedules evaluate exactly this expression, so they give the same bits and the choice may depend on the batch:
//   * two launches (lsm_partial_kernel + lsm_write_kernel): one work-group per segment; fills the chip for a handful
//     of rows, but reads the row twice (12 bytes moved per fp32 element for 8 algorithmic);
//   * one launch (lsm_resident_kernel): one work-group of 512 threads per row keeps the whole row on chip between the
//     read and the write -- 28 segments in registers (224 of the 256 registers of every thread), the rest in LDS --
//     so every element is read once and written once.  Rows of up to 154,624 elements fit (a 151,936-entry
//     vocabulary does).
// exp is 2^(d * log2 e) on the hardware exponential in both.
// ================================================================================================
constexpr int kSeg = 4096;  // elements per segment: 256 threads x 4 chunks x 4 floats
constexpr int kResidentRegSegs = 28;                          // segments a resident work-group holds in registers
constexpr int kResidentLdsFloats = (160 * 1024 - 4096) / 4;   // row elements it can hold in LDS behind those
constexpr int64_t kResidentMaxCols = (int64_t)kResidentRegSegs * kSeg + kResidentLdsFloats;

enum { LSM_F32 = 0, LSM_BF16 = 1, LSM_F16 = 2 };

struct LsmArgs {
  const void* x;
  void* out;
  float* ws;  // [rows][segs][2]
  int64_t ldx, ldo;
  int64_t rows, cols;
  int segs;
  int vec;  // rows allow full-width vector loads/stores of a 4-element chunk
  int write_softmax;
};

__device__ __forceinline__ float fast_exp(float d) { return __builtin_amdgcn_exp2f(d * 1.44269504088896340736f); }

template <int T>
struct LsmElem;
template <>
struct LsmElem<LSM_F32> {
  typedef float type;
  static __device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
    const float4 q = *reinterpret_cast<const float4*>(p);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  }
  static __device__ __forceinline__ float load1(const float* p) { return *p; }
  static __device__ __forceinline__ void store4(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
  static __device__ __forceinline__ void store1(float* p, float v) { *p = v; }
};
template <>
struct LsmElem<LSM_BF16> {
  typedef uint16_t type;
  static __device__ __forceinline__ void load4(const uint16_t* p, float (&v)[4]) {
    const uint2 q = *reinterpret_cast<const uint2*>(p);
    v[0] = bf16_lo(q.x); v[1] = bf16_hi(q.x); v[2] = bf16_lo(q.y); v[3] = bf16_hi(q.y);
  }
  static __device__ __forceinline__ float load1(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  static __device__ __forceinline__ void store4(uint16_t* p, const float (&v)[4]) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
  }
  static __device__ __forceinline__ void store1(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
};
template <>
struct LsmElem<LSM_F16> {
  typedef uint16_t type;
  static __device__ __forceinline__ void load4(const uint16_t* p, float (&v)[4]) {
    const uint2 q = *reinterpret_cast<const uint2*>(p);
    const f16x2 a = __builtin_bit_cast(f16x2, q.x), b = __builtin_bit_cast(f16x2, q.y);
    v[0] = (float)a[0]; v[1] = (float)a[1]; v[2] = (float)b[0]; v[3] = (float)b[1];
  }
  static __device__ __forceinline__ float load1(const uint16_t* p) { return f16_bits_to_f32(*p); }
  static __device__ __forceinline__ void store4(uint16_t* p, const float (&v)[4]) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_f16x2(v[0], v[1]), pack_f16x2(v[2], v[3]));
  }
  static __device__ __forceinline__ void store1(uint16_t* p, float v) { *p = (uint16_t)(pack_f16x2(v, 0.f) & 0xffffu); }
};

// The 4-element chunk that starts at element e of a row; out-of-range elements read as `fill`.
template <int IN>
__device__ __forceinline__ void load_chunk(const typename LsmElem<IN>::type* row, int64_t e, int64_t cols, int vec, float fill,
                                           float (&v)[4]) {
  if (vec && e + 3 < cols) {
    LsmElem<IN>::load4(row + e, v);
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = (e + j < cols) ? LsmElem<IN>::load1(row + e + j) : fill;
  }
}
template <int OUT>
__device__ __forceinline__ void store_chunk(typename LsmElem<OUT>::type* row, int64_t e, int64_t cols, int vec, const float (&v)[4]) {
  if (vec && e + 3 < cols) {
    LsmElem<OUT>::store4(row + e, v);
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (e + j < cols) LsmElem<OUT>::store1(row + e + j, v[j]);
  }
}

// Thread t (0..255) of a segment's team: its 16 elements (chunk q = t + 256*i holds elements 4q..4q+3 of the segment).
template <int IN>
__device__ __forceinline__ void load_seg(const typename LsmElem<IN>::type* row, int64_t base, int t, int64_t cols, int vec,
                                         float fill, float (&v)[4][4]) {
#pragma unroll
  for (int i = 0; i < 4; i++) load_chunk<IN>(row, base + 4 * (int64_t)(t + 256 * i), cols, vec, fill, v[i]);
}

__device__ __forceinline__ float seg_thread_max(const float (&v)[4][4]) {
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) m = fmaxf(m, v[i][j]);
  return m;
}
__device__ __forceinline__ float seg_thread_expsum(const float (&v)[4][4], float m) {
  // exp(x - m) = 2^((x - m) * log2 e): the difference is formed first (exact near the maximum, where the terms that
  // matter are), so a common offset of the logits does not enter the rounding; then the hardware exponential
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) s += fast_exp(v[i][j] - m);  // 2^(-inf) = 0 for the padding
  return s;
}

// The merge of a row's segment pairs by ONE wavefront: lane l takes segments l, l+64, ... in ascending order, then the
// fixed butterfly.  Returns (global max, log of the global sum) in every lane.
__device__ __forceinline__ void merge_segments(const float* w, int segs, int lane, float& gmax, float& lg) {
  float lm = -INFINITY;
  for (int s = lane; s < segs; s += 64) lm = fmaxf(lm, w[2 * s]);
  gmax = wave_max(lm);
  float ls = 0.f;
  for (int s = lane; s < segs; s += 64) ls += w[2 * s + 1] * expf(w[2 * s] - gmax);
  lg = logf(wave_sum(ls));
}

template <int IN>
__global__ __launch_bounds__(256) void lsm_partial_kernel(const LsmArgs a) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x / a.segs;
  const int seg = blockIdx.x % a.segs;
  const typename LsmElem<IN>::type* xr = static_cast<const typename LsmElem<IN>::type*>(a.x) + row * a.ldx;
  float v[4][4];
  load_seg<IN>(xr, (int64_t)seg * kSeg, threadIdx.x, a.cols, a.vec, -INFINITY, v);
  float m = wave_max(seg_thread_max(v));
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  const float s = wave_sum(seg_thread_expsum(v, m));
  if (lane == 0) red[wave] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float tot = ((red[0] + red[1]) + red[2]) + red[3];
    float* w = a.ws + ((int64_t)row * a.segs + seg) * 2;
    w[0] = m;
    w[1] = tot;
  }
}

template <int IN, int OUT>
__global__ __launch_bounds__(256) void lsm_write_kernel(const LsmArgs a) {
  const int64_t row = blockIdx.x / a.segs;
  const int seg = blockIdx.x % a.segs;
  // merged by the first wavefront only: the other 192 threads do not repeat the work
  __shared__ float stat[2];
  if (threadIdx.x < 64) {
    float gmax, lg;
    merge_segments(a.ws + (int64_t)row * a.segs * 2, a.segs, threadIdx.x, gmax, lg);
    if (threadIdx.x == 0) {
      stat[0] = gmax;
      stat[1] = lg;
    }
  }
  __syncthreads();
  const float gm = stat[0], lg = stat[1];
  const typename LsmElem<IN>::type* xr = static_cast<const typename LsmElem<IN>::type*>(a.x) + row * a.ldx;
  typename LsmElem<OUT>::type* orow = static_cast<typename LsmElem<OUT>::type*>(a.out) + row * a.ldo;
  float v[4][4];
  load_seg<IN>(xr, (int64_t)seg * kSeg, threadIdx.x, a.cols, a.vec, 0.f, v);
#pragma unroll
  for (int i = 0; i < 4; i++) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const float y = (v[i][j] - gm) - lg;
      v[i][j] = a.write_softmax ? fast_exp(y) : y;
    }
    store_chunk<OUT>(orow, (int64_t)seg * kSeg + 4 * (int64_t)(threadIdx.x + 256 * i), a.cols, a.vec, v[i]);
  }
}

// One work-group of 512 threads per row: its two halves are the 256-thread teams of two segments at a time
// (slot k = segments 2k and 2k+1).  The first 28 full segments stay in registers (14 slots of 16 values per thread),
// what follows (further full segments and the ragged last one) in LDS at its row offset.  Every reduction is the one
// of the two-launch schedule, value for value.  Rows must allow vector access (a.vec).  The code is kept small on
// purpose -- branch-free for full segments, run-time loops over the LDS part -- because it runs once per row and has
// to stay in the instruction cache.
template <int IN, int OUT, bool SOFTMAX>
__global__ __launch_bounds__(512) void lsm_resident_kernel(const LsmArgs a) {
  constexpr int RK = kResidentRegSegs / 2;  // register slots
  constexpr int MAXSEG = (int)((kResidentMaxCols + kSeg - 1) / kSeg);
  extern __shared__ __attribute__((aligned(16))) float lds_row[];   // [kResidentLdsFloats] row tail, then the statistics
  float* red = lds_row + kResidentLdsFloats;                        // [MAXSEG][4] wave partials of a segment
  float* stat = red + MAXSEG * 4;                                   // [MAXSEG][2] (max, sum) per segment, then 2 row values
  typedef typename LsmElem<IN>::type in_t;
  typedef typename LsmElem<OUT>::type out_t;
  const int tid = threadIdx.x, half = tid >> 8, t = tid & 255, lane = tid & 63, wave = (tid >> 6) & 3;
  // every XCD walks a contiguous range of rows (4096 rows of 151936 floats: 1026 -> 979 us)
  const int64_t row = xcd_contiguous_tile(blockIdx.x, gridDim.x);
  const in_t* xr = static_cast<const in_t*>(a.x) + row * a.ldx;
  out_t* orow = static_cast<out_t*>(a.out) + row * a.ldo;
  const int cols = (int)a.cols, segs = a.segs;
  const int nfull = cols >> 12;                                       // full segments
  const int nreg = (nfull & ~1) < 2 * RK ? (nfull & ~1) : 2 * RK;     // ... of which in registers (whole slots)
  const int nslot = nreg >> 1;
  const int lds0 = nreg * kSeg;                                       // first row element that lives in LDS
  const int t4 = 4 * t;
  const int mine = half * kSeg + t4;  // thread's chunk i of slot k starts at row element k*8192 + mine + 1024*i

  auto from_lds = [&](int sg, float (&u)[4][4]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int e = sg * kSeg + t4 + 1024 * i;
      if (e >= cols) {   // only in the ragged segment: chunks past the end of the row have no place in LDS
        u[i][0] = u[i][1] = u[i][2] = u[i][3] = -INFINITY;
      } else {
        const float4 q = *reinterpret_cast<const float4*>(lds_row + (e - lds0));
        u[i][0] = q.x; u[i][1] = q.y; u[i][2] = q.z; u[i][3] = q.w;
      }
    }
  };
  auto finish = [&](int e0, float (&u)[4][4], bool ragged) __attribute__((always_inline)) {
    const float gm = stat[2 * MAXSEG], lg = stat[2 * MAXSEG + 1];
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float y = (u[i][j] - gm) - lg;
        u[i][j] = SOFTMAX ? fast_exp(y) : y;
      }
      if (!ragged) LsmElem<OUT>::store4(orow + e0 + 1024 * i, u[i]);
      else store_chunk<OUT>(orow, e0 + 1024 * i, cols, 1, u[i]);
    }
  };

  // ---- read the row once.  The part that lives in LDS goes first, four segments per team and round trip through
  // registers that the register part does not occupy yet (one segment per round trip would cost a memory latency
  // each); the loads of the register part are then all in flight together and are consumed in order.
  constexpr int LB = 4;
  for (int sg0 = nreg + half; sg0 < segs; sg0 += 2 * LB) {
    float u[LB][4][4];
#pragma unroll
    for (int b = 0; b < LB; b++) {
      const int sg = sg0 + 2 * b;
      if (sg < nfull) {
#pragma unroll
        for (int i = 0; i < 4; i++) LsmElem<IN>::load4(xr + sg * kSeg + t4 + 1024 * i, u[b][i]);
      } else if (sg < segs) {   // the ragged last segment
#pragma unroll
        for (int i = 0; i < 4; i++) load_chunk<IN>(xr, sg * kSeg + t4 + 1024 * i, cols, 1, -INFINITY, u[b][i]);
      }
    }
#pragma unroll
    for (int b = 0; b < LB; b++) {
      const int sg = sg0 + 2 * b;
      if (sg < segs) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int e = sg * kSeg + t4 + 1024 * i;
          if (e < cols) *reinterpret_cast<float4*>(lds_row + (e - lds0)) = make_float4(u[b][i][0], u[b][i][1], u[b][i][2], u[b][i][3]);
        }
      }
    }
  }
  float v[RK][4][4];
#pragma unroll
  for (int k = 0; k < RK; k++)
    if (k < nslot) {
#pragma unroll
      for (int i = 0; i < 4; i++) LsmElem<IN>::load4(xr + k * 2 * kSeg + mine + 1024 * i, v[k][i]);
    }

  // ---- segment maxima: per thread, butterfly, then the four wavefronts of the team in order
#pragma unroll
  for (int k = 0; k < RK; k++)
    if (k < nslot) {
      const float m = wave_max(seg_thread_max(v[k]));
      if (lane == 0) red[(2 * k + half) * 4 + wave] = m;
    }
  for (int sg = nreg + half; sg < segs; sg += 2) {
    float u[4][4];
    from_lds(sg, u);
    const float m = wave_max(seg_thread_max(u));
    if (lane == 0) red[sg * 4 + wave] = m;
  }
  __syncthreads();
  if (tid < segs) stat[2 * tid] = fmaxf(fmaxf(red[4 * tid], red[4 * tid + 1]), fmaxf(red[4 * tid + 2], red[4 * tid + 3]));
  __syncthreads();
  // ---- segment sums of exp(x - segment max)
#pragma unroll
  for (int k = 0; k < RK; k++)
    if (k < nslot) {
      const float sm = wave_sum(seg_thread_expsum(v[k], stat[2 * (2 * k + half)]));
      if (lane == 0) red[(2 * k + half) * 4 + wave] = sm;
    }
  for (int sg = nreg + half; sg < segs; sg += 2) {
    float u[4][4];
    from_lds(sg, u);
    const float sm = wave_sum(seg_thread_expsum(u, stat[2 * sg]));
    if (lane == 0) red[sg * 4 + wave] = sm;
  }
  __syncthreads();
  if (tid < segs) stat[2 * tid + 1] = ((red[4 * tid] + red[4 * tid + 1]) + red[4 * tid + 2]) + red[4 * tid + 3];
  __syncthreads();
  // ---- the row's (max, log sum): first wavefront, as in the two-launch schedule
  if (tid < 64) {
    float gmax, lg;
    merge_segments(stat, segs, tid, gmax, lg);
    if (tid == 0) {
      stat[2 * MAXSEG] = gmax;
      stat[2 * MAXSEG + 1] = lg;
    }
  }
  __syncthreads();
  // ---- write the row once
#pragma unroll
  for (int k = 0; k < RK; k++)
    if (k < nslot) finish(k * 2 * kSeg + mine, v[k], false);
  for (int sg = nreg + half; sg < segs; sg += 2) {
    float u[4][4];
    from_lds(sg, u);
    if (sg < nfull) finish(sg * kSeg + t4, u, false);
    else finish(sg * kSeg + t4, u, true);
  }
}

// One launch with the row resident on chip once there are enough rows to occupy the CUs with one work-group each (same
// bits either way); that schedule does not touch the workspace.
static bool lsm_resident(int64_t rows, int64_t cols) { return cols <= kResidentMaxCols && rows >= 192; }

size_t lsm_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  const int64_t segs = (cols + kSeg - 1) / kSeg;
  return (size_t)rows * (size_t)segs * 2 * sizeof(float);
}

template <int IN, int OUT>
static int lsm_launch(const LsmArgs& a, bool resident, hipStream_t stream) {
  if (resident) {
    constexpr int lds = 160 * 1024;
    if (a.write_softmax) {
      static std::atomic<uint64_t> done{0};
      hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(lsm_resident_kernel<IN, OUT, true>), lds, done);
      if (e != hipSuccess) return hip_code(e);
      hipLaunchKernelGGL((lsm_resident_kernel<IN, OUT, true>), dim3((unsigned)a.rows), dim3(512), lds, stream, a);
    } else {
      static std::atomic<uint64_t> done{0};
      hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(lsm_resident_kernel<IN, OUT, false>), lds, done);
      if (e != hipSuccess) return hip_code(e);
      hipLaunchKernelGGL((lsm_resident_kernel<IN, OUT, false>), dim3((unsigned)a.rows), dim3(512), lds, stream, a);
    }
  } else {
    const dim3 grid((unsigned)(a.rows * a.segs)), block(256);
    hipLaunchKernelGGL((lsm_partial_kernel<IN>), grid, block, 0, stream, a);
    hipLaunchKernelGGL((lsm_write_kernel<IN, OUT>), grid, block, 0, stream, a);
  }
  return hip_code(hipGetLastError());
}

// dtype codes: 0 fp32, 1 bf16, 2 fp16; the output is fp32 or the input's type
int log_softmax_dispatch(const void* x, int64_t ldx, int in_dtype, void* out, int64_t ldo, int out_dtype, int64_t rows,
                         int64_t cols, void* ws, size_t ws_bytes, int write_softmax, hipStream_t stream) {
  if (rows < 0 || cols <= 0 || ldx < cols || ldo < cols) return TBIK_ERR_INVALID;
  if (in_dtype < 0 || in_dtype > 2 || (out_dtype != LSM_F32 && out_dtype != in_dtype)) return TBIK_ERR_UNSUPPORTED;
  if (rows == 0) return TBIK_OK;
  if (!x || !out) return TBIK_ERR_INVALID;
  const int isz = in_dtype == LSM_F32 ? 4 : 2, osz = out_dtype == LSM_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(x) & (isz - 1)) || (reinterpret_cast<uintptr_t>(out) & (osz - 1))) return TBIK_ERR_ALIGNMENT;
  const int64_t segs = (cols + kSeg - 1) / kSeg;
  if (rows * segs > 0x7fffffff) return TBIK_ERR_INVALID;
  // the vector and the scalar path read the same elements into the same registers: same order
  const int vec = ((reinterpret_cast<uintptr_t>(x) & (4 * isz - 1)) == 0 && (reinterpret_cast<uintptr_t>(out) & (4 * osz - 1)) == 0 &&
                   (ldx & 3) == 0 && (ldo & 3) == 0)
                      ? 1
                      : 0;
  const bool resident = vec && lsm_resident(rows, cols);
  if (!resident && (!ws || ws_bytes < lsm_workspace_bytes(rows, cols) || (reinterpret_cast<uintptr_t>(ws) & 3))) return TBIK_ERR_WORKSPACE;
  LsmArgs a;
  a.x = x;
  a.out = out;
  a.ws = static_cast<float*>(ws);
  a.ldx = ldx;
  a.ldo = ldo;
  a.rows = rows;
  a.cols = cols;
  a.segs = (int)segs;
  a.vec = vec;
  a.write_softmax = write_softmax;
  if (in_dtype == LSM_F32) return lsm_launch<LSM_F32, LSM_F32>(a, resident, stream);
  if (in_dtype == LSM_BF16)
    return out_dtype == LSM_F32 ? lsm_launch<LSM_BF16, LSM_F32>(a, resident, stream) : lsm_launch<LSM_BF16, LSM_BF16>(a, resident, stream);
  return out_dtype == LSM_F32 ? lsm_launch<LSM_F16, LSM_F32>(a, resident, stream) : lsm_launch<LSM_F16, LSM_F16>(a, resident, stream);
}

// ================================================================================================
// mean over the middle dimension of a contiguous (outer, n, inner) view.
// inner == 1: lane l of the row's team owns elements 4*(l + W*i) .. +3 (W = 64 lanes for n <= 8192,
//             256 threads above that); sequential inside a lane, butterfly across lanes, waves joined
//             in wave order.
// inner  > 1: one thread per output element walks n sequentially (loads coalesce along inner).
// Replaces mean_kernel, src/bio/batch_invariant_ops.py:304-349.
// ================================================================================================
template <typename T>
__device__ __forceinline__ float load_as_f32(const T* p);
template <>
__device__ __forceinline__ float load_as_f32<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }
template <>
__device__ __forceinline__ float load_as_f32<_Float16>(const _Float16* p) { return (float)*p; }

template <typename T>
__device__ __forceinline__ void store_from_f32(T* p, float v);
template <>
__device__ __forceinline__ void store_from_f32<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_from_f32<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
template <>
__device__ __forceinline__ void store_from_f32<_Float16>(_Float16* p, float v) { *p = (_Float16)v; }

template <typename T, int TEAM>  // TEAM = 64: one wave per row, 4 rows per block; TEAM = 256: block per row
__global__ __launch_bounds__(256) void mean_rows_kernel(const T* x, T* out, int64_t rows, int64_t n) {
  __shared__ float red[4];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t row = TEAM == 64 ? (int64_t)blockIdx.x * 4 + wave : (int64_t)blockIdx.x;
  const int member = TEAM == 64 ? lane : (int)threadIdx.x;
  float s = 0.f;
  if (row < rows) {
    const T* xr = x + row * n;
    const bool vec = sizeof(T) == 4 && ((reinterpret_cast<uintptr_t>(xr) & 15) == 0);
    for (int64_t e = 4 * (int64_t)member; e < n; e += 4 * TEAM) {
      if (vec && e + 3 < n) {
        const float4 q = *reinterpret_cast<const float4*>(xr + e);
        s += q.x; s += q.y; s += q.z; s += q.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (e + j < n) s += load_as_f32<T>(xr + e + j);
      }
    }
  }
  s = wave_sum(s);
  if (TEAM == 64) {
    if (row < rows && lane == 0) store_from_f32<T>(out + row, s / (float)n);
  } else {
    if (lane == 0) red[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0) store_from_f32<T>(out + row, (((red[0] + red[1]) + red[2]) + red[3]) / (float)n);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void mean_mid_kernel(const T* x, T* out, int64_t outer, int64_t n, int64_t inner) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= outer * inner) return;
  const int64_t o = idx / inner, k = idx % inner;
  const T* p = x + o * n * inner + k;
  float s = 0.f;
  for (int64_t i = 0; i < n; i++) s += load_as_f32<T>(p + i * inner);
  store_from_f32<T>(out + idx, s / (float)n);
}

template <typename T>
static int mean_launch(const void* x, void* out, int64_t outer, int64_t n, int64_t inner, hipStream_t stream) {
  const T* xp = static_cast<const T*>(x);
  T* op = static_cast<T*>(out);
  if (inner == 1) {
    if (n <= 8192) {
      const int64_t blocks = (outer + 3) / 4;
      if (blocks > 0x7fffffff) return TBIK_ERR_INVALID;
      hipLaunchKernelGGL((mean_rows_kernel<T, 64>), dim3((unsigned)blocks), dim3(256), 0, stream, xp, op, outer, n);
    } else {
      if (outer > 0x7fffffff) return TBIK_ERR_INVALID;
      hipLaunchKernelGGL((mean_rows_kernel<T, 256>), dim3((unsigned)outer), dim3(256), 0, stream, xp, op, outer, n);
    }
  } else {
    const int64_t blocks = (outer * inner + 255) / 256;
    if (blocks > 0x7fffffff) return TBIK_ERR_INVALID;
    hipLaunchKernelGGL(mean_mid_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream, xp, op, outer, n, inner);
  }
  return hip_code(hipGetLastError());
}

// ------------------------------------------------------------------------------------------------
// Greedy sampling: index of the largest element of each row, ties resolved to the lowest index (a NaN is never
// selected; a row of NaNs gives index 0).  "Largest value, then lowest index" is a total order on (value, index)
// pairs, so the result does not depend on how the row is cut over lanes and waves: batch invariant by construction.
// One work-group of 1024 threads per row, 16-byte packs of 8 bf16.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void argmax_take(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) {
    bv = v;
    bi = i;
  }
}

// Optional bookkeeping of a decode step, done by the work-group of a row once its index is known (all pointers may be
// null): the index also goes to history[row * history_ld + count[row]] (skipped when the row's history is full) and
// count[row], positions[row] and ctx_len[row] advance by one.
struct ArgmaxAdvance {
  int64_t* history;
  int64_t history_ld;
  int64_t* count;
  int64_t* positions;
  int* ctx_len;
};

__global__ __launch_bounds__(1024) void argmax_rows_kernel(const uint16_t* x, int64_t ld, int64_t* out, int cols, const ArgmaxAdvance adv) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const uint16_t* xr = x + (int64_t)blockIdx.x * ld;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  const bool vec = ((reinterpret_cast<uintptr_t>(xr) & 15) == 0);
  const int npacks = vec ? cols / 8 : 0;
  // eight packs in flight per thread (a pack past the end re-reads the last one and is skipped): one round trip
  // covers 64 Ki elements of the row.  A thread meets its elements in ascending index order, so inside the thread
  // "strictly larger" keeps the lowest index of equal values; the full (value, index) order is needed only across lanes.
  for (int q0 = tid; q0 < npacks; q0 += 8 * 1024) {
    uint4 pk[8];
#pragma unroll
    for (int u = 0; u < 8; u++) pk[u] = *reinterpret_cast<const uint4*>(xr + (int64_t)min(q0 + u * 1024, npacks - 1) * 8);
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const int q = q0 + u * 1024;
      if (q < npacks) {
        const uint32_t w[4] = {pk[u].x, pk[u].y, pk[u].z, pk[u].w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float lo = bf16_lo(w[e]), hi = bf16_hi(w[e]);
          if (lo > bv) { bv = lo; bi = q * 8 + 2 * e; }
          if (hi > bv) { bv = hi; bi = q * 8 + 2 * e + 1; }
        }
      }
    }
  }
  for (int i = npacks * 8 + tid; i < cols; i += 1024) argmax_take(bv, bi, bf16_bits_to_f32(xr[i]), i);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(bv, off);
    const int oi = __shfl_xor(bi, off);
    argmax_take(bv, bi, ov, oi);
  }
  if (lane == 0) {
    sv[wave] = bv;
    si[wave] = bi;
  }
  __syncthreads();
  if (tid == 0) {
#pragma unroll
    for (int w = 1; w < 16; w++) argmax_take(bv, bi, sv[w], si[w]);
    const int64_t idx = bi == 0x7fffffff ? 0 : bi;
    const int64_t r = blockIdx.x;
    out[r] = idx;
    if (adv.count) {
      const int64_t c = adv.count[r];
      if (adv.history && c >= 0 && c < adv.history_ld) adv.history[r * adv.history_ld + c] = idx;
      adv.count[r] = c + 1;
    }
    if (adv.positions) adv.positions[r] += 1;
    if (adv.ctx_len) adv.ctx_len[r] += 1;
  }
}

int argmax_dispatch(const void* x, int64_t ld, void* out, int64_t rows, int cols, void* history, int64_t history_ld,
                    void* count, void* positions, void* ctx_len, hipStream_t stream) {
  if (rows < 0 || cols <= 0 || ld < cols) return TBIK_ERR_INVALID;
  if (history && (!count || history_ld <= 0)) return TBIK_ERR_INVALID;
  if (rows == 0) return TBIK_OK;
  if (!x || !out || rows > 0x7fffffff) return TBIK_ERR_INVALID;
  auto mis = [](const void* p, uintptr_t m) { return (reinterpret_cast<uintptr_t>(p) & m) != 0; };
  if (mis(x, 1) || mis(out, 7) || mis(history, 7) || mis(count, 7) || mis(positions, 7) || mis(ctx_len, 3)) return TBIK_ERR_ALIGNMENT;
  const ArgmaxAdvance adv{static_cast<int64_t*>(history), history_ld, static_cast<int64_t*>(count),
                          static_cast<int64_t*>(positions), static_cast<int*>(ctx_len)};
  hipLaunchKernelGGL(argmax_rows_kernel, dim3((unsigned)rows), dim3(1024), 0, stream, static_cast<const uint16_t*>(x), ld,
                     static_cast<int64_t*>(out), cols, adv);
  return hip_code(hipGetLastError());
}

int mean_dispatch(const void* x, void* out, int64_t outer, int64_t n, int64_t inner, int dtype_code, hipStream_t stream) {
  if (outer < 0 || n <= 0 || inner <= 0) return TBIK_ERR_INVALID;
  if (outer == 0) return TBIK_OK;
  if (!x || !out) return TBIK_ERR_INVALID;
  switch (dtype_code) {
    case 0: return mean_launch<float>(x, out, outer, n, inner, stream);
    case 1: return mean_launch<uint16_t>(x, out, outer, n, inner, stream);
    case 2: return mean_launch<_Float16>(x, out, outer, n, inner, stream);
    default: return TBIK_ERR_UNSUPPORTED;
  }
}

}  // namespace tbik
