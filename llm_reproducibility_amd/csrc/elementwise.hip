// Gated activation feeding the row-split down projection: act[r, i] = silu(gu[r, i]) * gu[r, inter + i], bf16.
//
// This is the producer of the tree matmul's X operand (the MLP of the reference's models runs vLLM's
// SiluAndMul between the merged gate/up projection and down_proj, whose forward is the patched
// RowParallelLinear, src/patch/patch_tp_invariant.py:10-48).  Arithmetic: silu in fp32, rounded to bf16,
// then the product rounded to bf16 -- two roundings, as an unfused `F.silu(gate) * up` on bf16 tensors
// gives.  Elementwise, so batch invariant by construction.  HBM bound: 6 bytes per output element.
#include "common.h"

namespace tbik {

template <bool F16>
__device__ __forceinline__ uint32_t silu_mul_pair(uint32_t g, uint32_t u) {
  using Num = Num16<F16>;
  const float g0 = Num::lo(g), g1 = Num::hi(g);
  const float s0 = g0 / (1.0f + expf(-g0));
  const float s1 = g1 / (1.0f + expf(-g1));
  const uint32_t s = Num::pack(s0, s1);
  return Num::pack(Num::lo(s) * Num::lo(u), Num::hi(s) * Num::hi(u));
}

// One thread per 8 outputs (16-byte loads and stores); 2-D grid-stride over (row, pack).
template <bool F16>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* __restrict__ gu, int64_t ld_in,
                                                       uint16_t* __restrict__ out, int64_t ld_out, int64_t rows,
                                                       int packs_per_row, int inter) {
  const int64_t total = rows * packs_per_row;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / packs_per_row;
    const int c = (int)(i - r * packs_per_row) * 8;
    const uint4 g = *reinterpret_cast<const uint4*>(gu + r * ld_in + c);
    const uint4 u = *reinterpret_cast<const uint4*>(gu + r * ld_in + inter + c);
    uint4 o;
    o.x = silu_mul_pair<F16>(g.x, u.x);
    o.y = silu_mul_pair<F16>(g.y, u.y);
    o.z = silu_mul_pair<F16>(g.z, u.z);
    o.w = silu_mul_pair<F16>(g.w, u.w);
    *reinterpret_cast<uint4*>(out + r * ld_out + c) = o;
  }
}

int silu_mul_dispatch(const void* gate_up, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int inter, bool f16,
                      hipStream_t stream) {
  if (!gate_up || !out || rows < 0 || inter <= 0 || ld_in < 2 * (int64_t)inter || ld_out < inter) return TBIK_ERR_INVALID;
  if ((inter & 7) || (ld_in & 7) || (ld_out & 7)) return TBIK_ERR_ALIGNMENT;
  if ((reinterpret_cast<uintptr_t>(gate_up) & 15) || (reinterpret_cast<uintptr_t>(out) & 15)) return TBIK_ERR_ALIGNMENT;
  if (rows == 0) return TBIK_OK;
  const int packs = inter / 8;
  const int64_t blocks = (rows * packs + 255) / 256;
  const unsigned grid = (unsigned)(blocks < 16384 ? blocks : 16384);
  if (f16)
    hipLaunchKernelGGL(silu_mul_kernel<true>, dim3(grid), dim3(256), 0, stream, static_cast<const uint16_t*>(gate_up), ld_in,
                       static_cast<uint16_t*>(out), ld_out, rows, packs, inter);
  else
    hipLaunchKernelGGL(silu_mul_kernel<false>, dim3(grid), dim3(256), 0, stream, static_cast<const uint16_t*>(gate_up), ld_in,
                       static_cast<uint16_t*>(out), ld_out, rows, packs, inter);
  return hip_code(hipGetLastError());
}

}  // namespace tbik
