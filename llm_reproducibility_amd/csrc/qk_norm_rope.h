// Per-head RMSNorm + rotary embedding of ONE head (128 channels) by ONE wavefront, shared by the stand-alone kernel
// (elementwise.hip) and by the decode attention kernel that forms its own queries and the new key (attention.hip): one
// body, so both give the same bits.
//
// Lane l owns channels l and l + 64 (a rotary pair).  rmsnorm as in rmsnorm_row.h (fp32 statistics, the normalised
// value rounded to bf16, then a bf16 multiply by the weight); rope is rotate-half in fp32 with angle pos * inv_freq[l],
// rounded once to bf16.  Returns the two results packed (channel l in the low half, l + 64 in the high half).
#pragma once
#include "common.h"

namespace tbik {

__device__ __forceinline__ uint32_t qk_norm_rope_head(uint16_t r1, uint16_t r2, const uint16_t* w, int64_t pos,
                                                      const float* inv_freq, float eps, int lane) {
  // every product and sum is rounded on its own, except where a fused multiply-add is written out: left to the
  // compiler, a multiplication could be fused with the next addition in one kernel and not in the other
#pragma clang fp contract(off)
  const float x1 = bf16_bits_to_f32(r1), x2 = bf16_bits_to_f32(r2);
  const float ss = wave_sum(__builtin_fmaf(x1, x1, x2 * x2));
  const float rs = 1.0f / sqrtf(ss * (1.0f / 128.0f) + eps);
  const uint32_t nrm = pack_bf16x2(x1 * rs, x2 * rs);
  const uint32_t wv = pack_bf16x2(bf16_lo(nrm) * bf16_bits_to_f32(w[lane]), bf16_hi(nrm) * bf16_bits_to_f32(w[lane + 64]));
  const float y1 = bf16_lo(wv), y2 = bf16_hi(wv);
  const float ang = (float)pos * inv_freq[lane];
  const float c = cosf(ang), s = sinf(ang);
  return pack_bf16x2(y1 * c - y2 * s, y2 * c + y1 * s);
}

}  // namespace tbik
