// Shared device helpers for the gfx950 kernels: bf16 packing/rounding and wavefront reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

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
// One step combines every lane with lane ^ OFF.  The partner's value travels through VALU cross-lane moves
// (v_permlane32_swap / v_permlane16_swap for 32 and 16, DPP row rotate / quad permute for 8, 2 and 1) instead of
// an LDS permute (__shfl_xor), which costs a round trip through the LDS crossbar per step; only the step of 4 has
// no such move and keeps the permute.  Both operands of a step are the same pair as with __shfl_xor and the
// operations are commutative, so the bits do not change.
struct LaneSum { static __device__ __forceinline__ float f(float a, float b) { return a + b; } };
struct LaneMax { static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); } };
// the NaN-propagating maximum (v_maximum3_f32): equal to fmaxf unless an input is NaN, and one instruction where fmaxf
// first quiets inputs the compiler cannot prove quiet (MFMA results, lane exchanges)
struct LaneMaxNaN { static __device__ __forceinline__ float f(float a, float b) { return __builtin_elementwise_maximum(a, b); } };
template <int OFF, typename Op>
__device__ __forceinline__ float xor_step(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  if (OFF == 32) {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return Op::f(as_f32(r[0]), as_f32(r[1]));
  } else if (OFF == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return Op::f(as_f32(r[0]), as_f32(r[1]));
  } else if (OFF == 8) {
    return Op::f(v, as_f32(__builtin_amdgcn_update_dpp(0u, u, 0x128, 0xf, 0xf, false)));  // row_ror:8
  } else if (OFF == 2) {
    return Op::f(v, as_f32(__builtin_amdgcn_update_dpp(0u, u, 0x4e, 0xf, 0xf, false)));   // quad_perm [2,3,0,1]
  } else if (OFF == 1) {
    return Op::f(v, as_f32(__builtin_amdgcn_update_dpp(0u, u, 0xb1, 0xf, 0xf, false)));   // quad_perm [1,0,3,2]
  } else {
    return Op::f(v, __shfl_xor(v, OFF, kWave));
  }
}
template <typename Op>
__device__ __forceinline__ float wave_reduce(float v) {
  v = xor_step<32, Op>(v);
  v = xor_step<16, Op>(v);
  v = xor_step<8, Op>(v);
  v = xor_step<4, Op>(v);
  v = xor_step<2, Op>(v);
  return xor_step<1, Op>(v);
}
__device__ __forceinline__ float wave_sum(float v) { return wave_reduce<LaneSum>(v); }
__device__ __forceinline__ float wave_max(float v) { return wave_reduce<LaneMax>(v); }

inline int hip_code(hipError_t e) { return e == hipSuccess ? TBIK_OK : TBIK_ERR_HIP_BASE + (int)e; }

// Raises a kernel's dynamic-LDS limit the first time the kernel is launched on a device.  The limit is a property of
// the loaded function on that device, so setting it again on every launch only costs host time on the decode path.
// `done` is one flag word per kernel instantiation (a function-local static at the call site), one bit per device.
// Work-groups are handed to the eight XCDs round robin (work-group b runs on XCD b % 8).  This maps b to a tile index
// such that every XCD walks a contiguous range of the nwg tiles (ranges one longer on the first nwg % 8 XCDs): tiles
// that share operand rows meet in one L2, and a pass over a weight matrix is eight sequential streams.  Measured on a
// [128,4096] x [4096,151936] mm (594 tiles of 256 columns): 327 us with tile = b, 263 us with this map.
__device__ __forceinline__ int xcd_contiguous_tile(int b, int nwg) {
  const int q = nwg >> 3, r = nwg & 7, x = b & 7;
  return x * q + (x < r ? x : r) + (b >> 3);
}

inline hipError_t ensure_dynamic_lds(const void* kern, int bytes, std::atomic<uint64_t>& done) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    return hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  const uint64_t bit = 1ull << dev;
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}

}  // namespace tbik
