// silu(gate) * up on a packed pair of 16-bit elements, shared by the stand-alone kernel (elementwise.hip) and by the
// tree matmul that applies it while it stages its activations (gemm_tree_strip.hip): one body, so the same bits.
// silu in fp32, rounded to the element type, then the product rounded to the element type -- two roundings, as an
// unfused `F.silu(gate) * up` on 16-bit tensors gives.  silu(g) = g / d with d = 1 + 2^(-g * log2 e) on the hardware
// exponential, the quotient from the hardware reciprocal and one correction step (q = g * r; q += (g - d * q) * r: within
// half a unit in the last place of the exact g / d, like a division, which keeps the rounded silu on the host's side of
// a bf16 boundary in cases such as gate = 5.9375, whose silu lies 1.2 fp32 steps below one).  Seven instructions per
// element where the library division and expf take some twenty-five -- which matters when every work-group of a
// matmul forms its own copy of the activations.  The limits come out as they should: silu(0) = 0, silu(g) = g for
// large g, -0 for large negative g (d = inf: the correction is skipped there, it would be inf * 0).
#pragma once
#include "common.h"

namespace tbik {

__device__ __forceinline__ float silu_f32(float g) {
  constexpr float kNegLog2e = -1.44269504088896340736f;
  const float d = 1.0f + __builtin_amdgcn_exp2f(g * kNegLog2e);
  const float r = __builtin_amdgcn_rcpf(d);
  const float q = g * r;
  const float fixed = __builtin_fmaf(__builtin_fmaf(-d, q, g), r, q);
  return (d < 3.0e38f && __builtin_fabsf(g) < 3.0e38f) ? fixed : q;   // d = inf (gate below -88): q is -0 already; g = inf: q is inf
}

template <bool F16>
__device__ __forceinline__ uint32_t silu_mul_pair(uint32_t g, uint32_t u) {
  using Num = Num16<F16>;
  const float g0 = Num::lo(g), g1 = Num::hi(g);
  const float s0 = silu_f32(g0), s1 = silu_f32(g1);
  const uint32_t s = Num::pack(s0, s1);
  return Num::pack(Num::lo(s) * Num::lo(u), Num::hi(s) * Num::hi(u));
}

}  // namespace tbik
