// Ceiling probes for the benchmark: what this chip sustains on nothing but bf16 MFMAs (the ceiling of ANY bf16 matmul
// kernel on given operand data, below the nominal peak because the chip is power limited) and on a plain one-pass
// read of a buffer (the ceiling of the bandwidth-bound kernels).  They have no counterpart in the reference; they
// exist so that a roofline fraction can be read against a measured ceiling as well as against the published peak.
// They measure the machine, not the path: built into libtbik_measure.so, a library of its own that only the
// benchmark loads (declared in include/tbik_measure.h), and absent from libtbik_hip.so and its header.
#include "../csrc/common.h"
#include "../../include/tbik_measure.h"

namespace tbik {

// One work-group per CU (the launch requests 100 KiB of dynamic LDS, which keeps a second one out), WAVES wavefronts each with a 4x4 block of 16x16
// accumulators, the shape of the 64x64 wave tile of the tree GEMM.  Operands come from `src` (4096 x 16 bytes) once
// and stay in registers: no loads, no LDS, no other instruction in the loop.
template <int ORDER>  // 0: tiles row by row; 1: rows in alternating directions, so that every MFMA changes ONE operand
__global__ __launch_bounds__(512) void probe_mfma_kernel(const bf16x8* __restrict__ src, float* __restrict__ out, int iters) {
  f32x4 acc[4][4];
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = src[(threadIdx.x + 512 * i) & 4095];
    b[i] = src[(threadIdx.x + 512 * (i + 4)) & 4095];
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int jj = 0; jj < 4; jj++) {
        const int j = (ORDER == 1 && (i & 1)) ? 3 - jj : jj;
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
      }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) s += acc[i][j][0] + acc[i][j][3];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Grid-stride pass of 16-byte loads over `n16` words; every thread folds what it read into one word it writes out.
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, int64_t n16, uint32_t* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  uint32_t h = 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) {
    const uint4 v = src[i];
    h ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = h;
}

int probe_mfma_dispatch(const void* operands, void* out, int work_groups, int waves, int iters, hipStream_t stream) {
  if (!operands || !out || work_groups <= 0 || iters == 0 || (waves != 4 && waves != 8)) return TBIK_ERR_INVALID;
  if (reinterpret_cast<uintptr_t>(operands) & 15) return TBIK_ERR_ALIGNMENT;
  constexpr int lds = 100 * 1024;
  static std::atomic<uint64_t> done{0};
  static std::atomic<uint64_t> done1{0};
  const bool snake = iters < 0;   // a negative count selects the alternating tile order
  if (snake) iters = -iters;
  hipError_t e = snake ? ensure_dynamic_lds(reinterpret_cast<const void*>(probe_mfma_kernel<1>), lds, done1)
                       : ensure_dynamic_lds(reinterpret_cast<const void*>(probe_mfma_kernel<0>), lds, done);
  if (e != hipSuccess) return hip_code(e);
  if (snake)
    hipLaunchKernelGGL(probe_mfma_kernel<1>, dim3((unsigned)work_groups), dim3(64 * waves), lds, stream,
                       static_cast<const bf16x8*>(operands), static_cast<float*>(out), iters);
  else
    hipLaunchKernelGGL(probe_mfma_kernel<0>, dim3((unsigned)work_groups), dim3(64 * waves), lds, stream,
                       static_cast<const bf16x8*>(operands), static_cast<float*>(out), iters);
  return hip_code(hipGetLastError());
}

int probe_read_dispatch(const void* src, int64_t bytes, void* out, int work_groups, hipStream_t stream) {
  if (!src || !out || bytes < 16 || work_groups <= 0) return TBIK_ERR_INVALID;
  if (reinterpret_cast<uintptr_t>(src) & 15) return TBIK_ERR_ALIGNMENT;
  hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)work_groups), dim3(256), 0, stream, static_cast<const uint4*>(src),
                     bytes / 16, static_cast<uint32_t*>(out));
  return hip_code(hipGetLastError());
}

}  // namespace tbik

extern "C" {

int tbik_probe_mfma_bf16(const void* operands, void* out, int work_groups, int waves, int iters, void* stream) {
  return tbik::probe_mfma_dispatch(operands, out, work_groups, waves, iters, static_cast<hipStream_t>(stream));
}

int tbik_probe_read(const void* src, int64_t bytes, void* out, int work_groups, void* stream) {
  return tbik::probe_read_dispatch(src, bytes, out, work_groups, static_cast<hipStream_t>(stream));
}

}  // extern "C"
