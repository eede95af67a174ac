// Gated activation feeding the row-split down projection: act[r, i] = silu(gu[r, i]) * gu[r, inter + i], bf16.
//
// This is the producer of the tree matmul's X operand (the MLP of the reference's models runs vLLM's
// SiluAndMul between the merged gate/up projection and down_proj, whose forward is the patched
// RowParallelLinear, src/patch/patch_tp_invariant.py:10-48).  Arithmetic: silu in fp32, rounded to bf16,
// then the product rounded to bf16 -- two roundings, as an unfused `F.silu(gate) * up` on bf16 tensors
// gives.  Elementwise, so batch invariant by construction.  HBM bound: 6 bytes per output element.
#include "common.h"
#include "qk_norm_rope.h"
#include "silu_mul.h"

namespace tbik {


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
  if (rows < 0 || inter <= 0 || ld_in < 2 * (int64_t)inter || ld_out < inter) return TBIK_ERR_INVALID;
  if (rows == 0 && !(inter & 7)) return TBIK_OK;
  if (!gate_up || !out) return TBIK_ERR_INVALID;
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

namespace tbik {

// ------------------------------------------------------------------------------------------------
// Per-head q/k RMSNorm + rotary embedding + KV-cache write for a Qwen3-style attention block, one wavefront per
// (token, head) of the fused qkv projection output [tokens, (Hq + 2*Hkv) * 128]:
//   query heads : q_out[token, h, :]          = rope(rmsnorm(q) * q_weight)
//   key heads   : k_cache[seq, h, pos, :]      = rope(rmsnorm(k) * k_weight)
//   value heads : vt_cache[seq, h, :, pos]     = v                    (the attention kernel reads V transposed)
// rmsnorm as in rmsnorm_kernel (fp32 statistics, the normalised value rounded to bf16, then a bf16 multiply by the
// weight); rope is rotate-half in fp32 with angle pos * inv_freq[i], rounded once to bf16.  Everything is per
// (token, head): batch invariant by construction.  Lane l owns channels l and l + 64 (a rotary pair).
// This is the caller side of the fixed-order attention (the reference patches vLLM's rotary embedding and leaves the
// rest to the engine, src/patch/patch_training_inference_align.py:35-44).
// ------------------------------------------------------------------------------------------------
struct QkRopeArgs {
  const uint16_t* qkv;
  int64_t ld;
  const uint16_t* qw;
  const uint16_t* kw;
  const float* inv_freq;   // [64]
  const int64_t* pos;      // [tokens]
  const int64_t* seq;      // [tokens]
  uint16_t* q_out;         // [tokens, Hq, 128]
  uint16_t* k_cache;       // [B, Hkv, L, 128]
  uint16_t* vt_cache;      // [B, Hkv, 128, L]
  int64_t tokens;
  int q_heads, kv_heads, max_len, batch;
  float eps;
};

__global__ __launch_bounds__(256) void qk_norm_rope_cache_kernel(const QkRopeArgs a) {
  const int lane = threadIdx.x & 63;
  const int heads = a.q_heads + 2 * a.kv_heads;
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= a.tokens * heads) return;
  const int64_t tok = unit / heads;
  const int hh = (int)(unit % heads);
  const uint16_t* src = a.qkv + tok * a.ld + (int64_t)hh * 128;
  const uint16_t r1 = src[lane], r2 = src[lane + 64];
  const int64_t pos = a.pos[tok];
  const int64_t sq = a.seq[tok];
  if (hh >= a.q_heads + a.kv_heads) {  // value head: transposed store
    const int h = hh - a.q_heads - a.kv_heads;
    if (sq < 0 || sq >= a.batch || pos < 0 || pos >= a.max_len) return;
    uint16_t* dst = a.vt_cache + ((sq * a.kv_heads + h) * 128) * (int64_t)a.max_len + pos;
    dst[(int64_t)lane * a.max_len] = r1;
    dst[(int64_t)(lane + 64) * a.max_len] = r2;
    return;
  }
  const bool is_q = hh < a.q_heads;
  const uint16_t* w = is_q ? a.qw : a.kw;
  const uint32_t o = qk_norm_rope_head(r1, r2, w, pos, a.inv_freq, a.eps, lane);
  uint16_t* dst;
  if (is_q) {
    dst = a.q_out + (tok * a.q_heads + hh) * 128;
  } else {
    if (sq < 0 || sq >= a.batch || pos < 0 || pos >= a.max_len) return;
    dst = a.k_cache + (((sq * a.kv_heads + (hh - a.q_heads)) * (int64_t)a.max_len) + pos) * 128;
  }
  dst[lane] = (uint16_t)(o & 0xffffu);
  dst[lane + 64] = (uint16_t)(o >> 16);
}

int qk_norm_rope_cache_dispatch(const void* qkv, int64_t ld, const void* q_weight, const void* k_weight,
                                const float* inv_freq, const int64_t* positions, const int64_t* seq_of_token, void* q_out,
                                void* k_cache, void* vt_cache, int64_t tokens, int q_heads, int kv_heads, int head_dim,
                                int max_len, int batch, float eps, hipStream_t stream) {
  if (!qkv || !q_weight || !k_weight || !inv_freq || !positions || !seq_of_token || !q_out || !k_cache || !vt_cache)
    return TBIK_ERR_INVALID;
  if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || max_len <= 0 || batch <= 0) return TBIK_ERR_INVALID;
  if (head_dim != 128) return TBIK_ERR_UNSUPPORTED;
  if (ld < (int64_t)(q_heads + 2 * kv_heads) * 128) return TBIK_ERR_INVALID;
  if (tokens == 0) return TBIK_OK;
  const int64_t units = tokens * (q_heads + 2 * kv_heads);
  const int64_t blocks = (units + 3) / 4;
  if (blocks > 0x7fffffff) return TBIK_ERR_INVALID;
  QkRopeArgs a{static_cast<const uint16_t*>(qkv), ld, static_cast<const uint16_t*>(q_weight),
               static_cast<const uint16_t*>(k_weight), inv_freq, positions, seq_of_token, static_cast<uint16_t*>(q_out),
               static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(vt_cache), tokens, q_heads, kv_heads, max_len, batch, eps};
  hipLaunchKernelGGL(qk_norm_rope_cache_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return hip_code(hipGetLastError());
}

}  // namespace tbik
