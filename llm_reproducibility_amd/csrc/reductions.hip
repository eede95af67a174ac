// Batch-invariant row reductions for gfx950: RMSNorm (bf16 or fp16), log_softmax / softmax (fp32), mean.
//
// Rule shared by all kernels here: the decomposition of a row into lanes, wavefronts and segments,
// and the order in which partial sums meet, is a function of the ROW LENGTH only.  The number of rows
// only changes how many identical work-groups are launched.  No atomics, no split decided at run time.
#include "common.h"

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
  using Num = Num16<F16>;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  const int nchunks = a.hidden >> 3;
  const uint4* xr = reinterpret_cast<const uint4*>(a.x + row * a.ldx);
  const uint4* rr = a.res ? reinterpret_cast<const uint4*>(a.res + row * a.ldr) : nullptr;

  // the weights do not depend on the row: fetched together with it, not after the reduction (with a single row
  // the kernel is nothing but memory round trips in a chain)
  const uint4* wr = reinterpret_cast<const uint4*>(a.w);
  uint4 wq[CPL];
  if (wr) {
#pragma unroll
    for (int i = 0; i < CPL; i++) {
      const int c = lane + 64 * i;
      if (c < nchunks) wq[i] = wr[c];
    }
  }

  // all loads of the row go out before the first store: the residual output may alias the inputs as far as the
  // compiler knows, and loads issued behind a store would wait for one memory round trip per chunk
  uint4 xq[CPL], rq[CPL];
#pragma unroll
  for (int i = 0; i < CPL; i++) {
    const int c = lane + 64 * i;
    if (c < nchunks) {
      xq[i] = xr[c];
      if (rr) rq[i] = rr[c];
    }
  }
  float v[CPL][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < CPL; i++) {
    const int c = lane + 64 * i;
    if (c < nchunks) {
      const uint32_t u[4] = {xq[i].x, xq[i].y, xq[i].z, xq[i].w};
#pragma unroll
      for (int e = 0; e < 4; e++) {
        v[i][2 * e] = Num::lo(u[e]);
        v[i][2 * e + 1] = Num::hi(u[e]);
      }
      if (rr) {
        const uint32_t ru[4] = {rq[i].x, rq[i].y, rq[i].z, rq[i].w};
        uint32_t so[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          v[i][2 * e] += Num::lo(ru[e]);
          v[i][2 * e + 1] += Num::hi(ru[e]);
          so[e] = Num::pack(v[i][2 * e], v[i][2 * e + 1]);
        }
        if (a.res_out) reinterpret_cast<uint4*>(a.res_out + row * a.ldro)[c] = make_uint4(so[0], so[1], so[2], so[3]);
      }
#pragma unroll
      for (int e = 0; e < 8; e++) ss = fmaf(v[i][e], v[i][e], ss);
    }
  }
  ss = wave_sum(ss);
  const float var = ss / (float)a.hidden;
  const float rs = 1.0f / sqrtf(var + a.eps);
  uint4* orow = reinterpret_cast<uint4*>(a.out + row * a.ldo);
#pragma unroll
  for (int i = 0; i < CPL; i++) {
    const int c = lane + 64 * i;
    if (c < nchunks) {
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; e++) o[e] = Num::pack(v[i][2 * e] * rs, v[i][2 * e + 1] * rs);
      if (wr) {
        const uint32_t wu[4] = {wq[i].x, wq[i].y, wq[i].z, wq[i].w};
#pragma unroll
        for (int e = 0; e < 4; e++)
          o[e] = Num::pack(Num::lo(o[e]) * Num::lo(wu[e]), Num::hi(o[e]) * Num::hi(wu[e]));
      }
      orow[c] = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
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
// log_softmax / softmax over the last dimension, fp32.
// A row is cut into fixed segments of 4096 elements; kernel 1 reduces each segment to (max, sum of
// exp(x - max)); kernel 2 merges a row's segment pairs in segment order and writes the result.
// Replaces the one-program-per-row three-pass kernel of the reference
// (src/bio/batch_invariant_ops.py:200-260): rows no longer limit the parallelism, yet the per-row
// order stays a function of `cols` alone.
// ================================================================================================
constexpr int kSeg = 4096;  // elements per segment: 256 threads x 4 chunks x 4 floats

struct LsmArgs {
  const float* x;
  float* out;
  float* ws;  // [rows][segs][2]
  int64_t ldx, ldo;
  int64_t rows, cols;
  int segs;
  int vec;  // rows allow 16-byte loads/stores
  int write_softmax;
};

// Loads this thread's 16 elements of the segment (chunk q = tid + 256*i holds elements 4q..4q+3 of the
// segment); out-of-range elements read as `fill`.
__device__ __forceinline__ void load_seg(const float* row, int64_t base, int64_t cols, int vec, float fill,
                                         float (&v)[4][4]) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int64_t e = base + 4 * (int64_t)(threadIdx.x + 256 * i);
    if (vec && e + 3 < cols) {
      const float4 q = *reinterpret_cast<const float4*>(row + e);
      v[i][0] = q.x; v[i][1] = q.y; v[i][2] = q.z; v[i][3] = q.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) v[i][j] = (e + j < cols) ? row[e + j] : fill;
    }
  }
}

__global__ __launch_bounds__(256) void lsm_partial_kernel(const LsmArgs a) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x / a.segs;
  const int seg = blockIdx.x % a.segs;
  const float* xr = a.x + row * a.ldx;
  float v[4][4];
  load_seg(xr, (int64_t)seg * kSeg, a.cols, a.vec, -INFINITY, v);
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) m = fmaxf(m, v[i][j]);
  m = wave_max(m);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) s += expf(v[i][j] - m);  // exp(-inf) = 0 for the padding
  s = wave_sum(s);
  if (lane == 0) red[wave] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float tot = ((red[0] + red[1]) + red[2]) + red[3];
    float* w = a.ws + ((int64_t)row * a.segs + seg) * 2;
    w[0] = m;
    w[1] = tot;
  }
}

__global__ __launch_bounds__(256) void lsm_write_kernel(const LsmArgs a) {
  const int64_t row = blockIdx.x / a.segs;
  const int seg = blockIdx.x % a.segs;
  // The row's segment pairs are merged by the first wavefront only (lane l takes segments l, l+64, ... in
  // ascending order, then a fixed butterfly): the order is a function of `segs` alone, and the other 192
  // threads do not repeat the work.
  __shared__ float stat[2];
  if (threadIdx.x < 64) {
    const float* w = a.ws + (int64_t)row * a.segs * 2;
    float lm = -INFINITY;
    for (int s = threadIdx.x; s < a.segs; s += 64) lm = fmaxf(lm, w[2 * s]);
    const float gmax = wave_max(lm);
    float ls = 0.f;
    for (int s = threadIdx.x; s < a.segs; s += 64) ls += w[2 * s + 1] * expf(w[2 * s] - gmax);
    const float gsum = wave_sum(ls);
    if (threadIdx.x == 0) {
      stat[0] = gmax;
      stat[1] = logf(gsum);
    }
  }
  __syncthreads();
  const float gm = stat[0], lg = stat[1];
  const float* xr = a.x + row * a.ldx;
  float* orow = a.out + row * a.ldo;
  float v[4][4];
  load_seg(xr, (int64_t)seg * kSeg, a.cols, a.vec, 0.f, v);
#pragma unroll
  for (int i = 0; i < 4; i++) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float y = (v[i][j] - gm) - lg;
      v[i][j] = a.write_softmax ? expf(y) : y;
    }
    const int64_t e = (int64_t)seg * kSeg + 4 * (int64_t)(threadIdx.x + 256 * i);
    if (a.vec && e + 3 < a.cols) {
      *reinterpret_cast<float4*>(orow + e) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (e + j < a.cols) orow[e + j] = v[i][j];
    }
  }
}

size_t lsm_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  const int64_t segs = (cols + kSeg - 1) / kSeg;
  return (size_t)rows * (size_t)segs * 2 * sizeof(float);
}

int log_softmax_dispatch(const void* x, int64_t ldx, void* out, int64_t ldo, int64_t rows, int64_t cols, void* ws,
                         size_t ws_bytes, int write_softmax, hipStream_t stream) {
  if (rows < 0 || cols <= 0 || ldx < cols || ldo < cols) return TBIK_ERR_INVALID;
  if (rows == 0) return TBIK_OK;
  if (!x || !out) return TBIK_ERR_INVALID;
  if ((reinterpret_cast<uintptr_t>(x) & 3) || (reinterpret_cast<uintptr_t>(out) & 3)) return TBIK_ERR_ALIGNMENT;
  if (!ws || ws_bytes < lsm_workspace_bytes(rows, cols) || (reinterpret_cast<uintptr_t>(ws) & 3)) return TBIK_ERR_WORKSPACE;
  const int64_t segs = (cols + kSeg - 1) / kSeg;
  if (rows * segs > 0x7fffffff) return TBIK_ERR_INVALID;
  LsmArgs a;
  a.x = static_cast<const float*>(x);
  a.out = static_cast<float*>(out);
  a.ws = static_cast<float*>(ws);
  a.ldx = ldx;
  a.ldo = ldo;
  a.rows = rows;
  a.cols = cols;
  a.segs = (int)segs;
  // the vector and the scalar path read the same elements into the same registers: same order
  a.vec = ((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (ldx & 3) == 0 &&
           (ldo & 3) == 0)
              ? 1
              : 0;
  a.write_softmax = write_softmax;
  const dim3 grid((unsigned)(rows * segs)), block(256);
  hipLaunchKernelGGL(lsm_partial_kernel, grid, block, 0, stream, a);
  hipLaunchKernelGGL(lsm_write_kernel, grid, block, 0, stream, a);
  return hip_code(hipGetLastError());
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

__global__ __launch_bounds__(1024) void argmax_rows_kernel(const uint16_t* x, int64_t ld, int64_t* out, int cols) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const uint16_t* xr = x + (int64_t)blockIdx.x * ld;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  const bool vec = ((reinterpret_cast<uintptr_t>(xr) & 15) == 0);
  const int npacks = vec ? cols / 8 : 0;
  // eight packs in flight per thread (a pack past the end re-reads the last one and is skipped): one round trip
  // covers 64 Ki elements of the row
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
          argmax_take(bv, bi, bf16_lo(w[e]), q * 8 + 2 * e);
          argmax_take(bv, bi, bf16_hi(w[e]), q * 8 + 2 * e + 1);
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
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

int argmax_dispatch(const void* x, int64_t ld, void* out, int64_t rows, int cols, hipStream_t stream) {
  if (rows < 0 || cols <= 0 || ld < cols) return TBIK_ERR_INVALID;
  if (rows == 0) return TBIK_OK;
  if (!x || !out || rows > 0x7fffffff) return TBIK_ERR_INVALID;
  if ((reinterpret_cast<uintptr_t>(x) & 1) || (reinterpret_cast<uintptr_t>(out) & 7)) return TBIK_ERR_ALIGNMENT;
  hipLaunchKernelGGL(argmax_rows_kernel, dim3((unsigned)rows), dim3(1024), 0, stream, static_cast<const uint16_t*>(x), ld,
                     static_cast<int64_t*>(out), cols);
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
