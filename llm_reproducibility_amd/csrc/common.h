// Shared device helpers for the gfx950 kernels: bf16 packing/rounding and wavefront reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tbik_hip.h"

namespace tbik {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int kWave = 64;

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// Two fp32 -> two bf16 (round to nearest even, one v_cvt_pk_bf16_f32); `lo` lands in bits 0..15.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf16_lo(uint32_t p) { return as_f32(p << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t p) { return as_f32(p & 0xffff0000u); }

// One tree node on a packed pair: bf16 + bf16 -> bf16.  The fp32 sum of two bf16 values followed by
// one rounding equals the correctly rounded bf16 sum (24 >= 2*8+2 significand bits).
__device__ __forceinline__ uint32_t add_bf16x2(uint32_t a, uint32_t b) {
  return pack_bf16x2(bf16_lo(a) + bf16_lo(b), bf16_hi(a) + bf16_hi(b));
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return (uint16_t)(pack_bf16x2(f, 0.0f) & 0xffffu); }
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return as_f32(((uint32_t)h) << 16); }

// fp16 counterparts.  Two fp32 -> two fp16, round to nearest even; a tree node is one packed fp16 add (a single
// rounding of the exact sum, which is also what an fp32 add followed by a rounding to fp16 gives).
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
__device__ __forceinline__ uint32_t add_f16x2(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, a) + __builtin_bit_cast(f16x2, b));
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

// Arithmetic of the two 16-bit element types the GEMM kernels are instantiated for.
template <bool F16>
struct Num16;
template <>
struct Num16<false> {
  static __device__ __forceinline__ f32x4 mfma(const bf16x8& a, const bf16x8& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pack_bf16x2(lo, hi); }
  static __device__ __forceinline__ uint32_t add(uint32_t a, uint32_t b) { return add_bf16x2(a, b); }
  static __device__ __forceinline__ float to_f32(uint16_t h) { return bf16_bits_to_f32(h); }
  static __device__ __forceinline__ float lo(uint32_t p) { return bf16_lo(p); }
  static __device__ __forceinline__ float hi(uint32_t p) { return bf16_hi(p); }
};
template <>
struct Num16<true> {
  static __device__ __forceinline__ f32x4 mfma(const bf16x8& a, const bf16x8& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pack_f16x2(lo, hi); }
  static __device__ __forceinline__ uint32_t add(uint32_t a, uint32_t b) { return add_f16x2(a, b); }
  static __device__ __forceinline__ float to_f32(uint16_t h) { return f16_bits_to_f32(h); }
  static __device__ __forceinline__ float lo(uint32_t p) { return (float)__builtin_bit_cast(f16x2, p)[0]; }
  static __device__ __forceinline__ float hi(uint32_t p) { return (float)__builtin_bit_cast(f16x2, p)[1]; }
};

// Butterfly reductions over the 64 lanes of a wavefront.  The exchange pattern is fixed, so the
// association order of the sum is a constant of the kernel: it cannot depend on the launch.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

inline int hip_code(hipError_t e) { return e == hipSuccess ? TBIK_OK : TBIK_ERR_HIP_BASE + (int)e; }

}  // namespace tbik
