// Shard combine: out[i] = adjacent-pair binary tree over up to 32 bf16 (or fp16) partials, every node rounded to
// the element type.  This is the arithmetic of the reference's cross-GPU tree all-reduce
// (src/tbik/tree_based_all_reduce.py:32-37; packed_tree_reduce,
// mini_allreduce/tbik_kernel/csrc/allreduce/custom_all_reduce.cuh:203-234) applied to partials that
// already sit in one GPU's memory.  HBM bound: (nparts + 1) * numel * 2 bytes.
#include "common.h"

namespace tbik {

struct CombineArgs {
  const uint16_t* parts[32];
  uint16_t* out;
  int64_t numel;
  const uint16_t* bias;  // optional [ncols] row vector added (in bf16) after the tree; element i is in column i % ncols
  int ncols;
  int64_t ldo;           // 0: `out` is contiguous like the partials; else element i goes to out[(i / ncols) * ldo + i % ncols]
};

template <int NP, bool F16>
__device__ __forceinline__ uint32_t tree_node(const uint32_t (&v)[NP]) {
  uint32_t w[NP];
#pragma unroll
  for (int i = 0; i < NP; i++) w[i] = v[i];
#pragma unroll
  for (int step = 1; step < NP; step <<= 1)
#pragma unroll
    for (int left = 0; left < NP; left += 2 * step) w[left] = Num16<F16>::add(w[left], w[left + step]);
  return w[0];
}

// One thread per 16-byte pack (8 bf16); grid-stride so any numel fits one launch.
template <int NP, bool F16>
__global__ __launch_bounds__(256) void combine_vec_kernel(const CombineArgs a, int64_t npacks) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < npacks; i += stride) {
    uint4 in[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) in[p] = reinterpret_cast<const uint4*>(a.parts[p])[i];
    uint4 o;
    uint32_t v[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) v[p] = in[p].x;
    o.x = tree_node<NP, F16>(v);
#pragma unroll
    for (int p = 0; p < NP; p++) v[p] = in[p].y;
    o.y = tree_node<NP, F16>(v);
#pragma unroll
    for (int p = 0; p < NP; p++) v[p] = in[p].z;
    o.z = tree_node<NP, F16>(v);
#pragma unroll
    for (int p = 0; p < NP; p++) v[p] = in[p].w;
    o.w = tree_node<NP, F16>(v);
    if (a.bias) {  // ncols % 8 == 0 on this path: the pack stays inside one row
      const uint4 bq = *reinterpret_cast<const uint4*>(a.bias + (i * 8) % a.ncols);
      o.x = Num16<F16>::add(o.x, bq.x);
      o.y = Num16<F16>::add(o.y, bq.y);
      o.z = Num16<F16>::add(o.z, bq.z);
      o.w = Num16<F16>::add(o.w, bq.w);
    }
    if (a.ldo) {  // ncols % 8 == 0 and aligned rows on this path
      const int64_t e = i * 8, r = e / a.ncols;
      *reinterpret_cast<uint4*>(a.out + r * a.ldo + (e - r * a.ncols)) = o;
    } else {
      reinterpret_cast<uint4*>(a.out)[i] = o;
    }
  }
}

// Scalar path for the tail and for buffers that are not 16-byte aligned.
template <int NP, bool F16>
__global__ __launch_bounds__(256) void combine_scalar_kernel(const CombineArgs a, int64_t begin) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = begin + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.numel; i += stride) {
    uint32_t v[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) v[p] = a.parts[p][i];
    uint32_t r = tree_node<NP, F16>(v);
    if (a.bias) r = Num16<F16>::add(r, a.bias[i % a.ncols]);
    const int64_t o = a.ldo ? (i / a.ncols) * a.ldo + i % a.ncols : i;
    a.out[o] = (uint16_t)(r & 0xffffu);
  }
}

template <int NP, bool F16>
static int launch_combine(const CombineArgs& a, bool vec_ok, hipStream_t stream) {
  const int64_t npacks = vec_ok ? a.numel / 8 : 0;
  if (npacks > 0) {
    const int64_t blocks = (npacks + 255) / 256;
    const unsigned grid = (unsigned)(blocks < 8192 ? blocks : 8192);
    hipLaunchKernelGGL((combine_vec_kernel<NP, F16>), dim3(grid), dim3(256), 0, stream, a, npacks);
  }
  const int64_t begin = npacks * 8;
  if (begin < a.numel) {
    const int64_t rest = a.numel - begin;
    const int64_t blocks = (rest + 255) / 256;
    const unsigned grid = (unsigned)(blocks < 8192 ? blocks : 8192);
    hipLaunchKernelGGL((combine_scalar_kernel<NP, F16>), dim3(grid), dim3(256), 0, stream, a, begin);
  }
  return hip_code(hipGetLastError());
}

int tree_combine_bias_dispatch(const void* const* parts, int nparts, void* out, int64_t numel, const void* bias, int N,
                               bool f16, hipStream_t stream, int64_t ldo) {
  if (numel < 0 || ((bias || ldo) && N <= 0) || (ldo && ldo < N)) return TBIK_ERR_INVALID;
  if (ldo == N) ldo = 0;
  if (nparts < 1 || nparts > 32 || (nparts & (nparts - 1))) return TBIK_ERR_INVALID;
  if (numel == 0) return TBIK_OK;
  if (!parts || !out) return TBIK_ERR_INVALID;
  CombineArgs a;
  bool vec_ok = (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  if (reinterpret_cast<uintptr_t>(out) & 1) return TBIK_ERR_ALIGNMENT;
  for (int p = 0; p < 32; p++) a.parts[p] = nullptr;
  for (int p = 0; p < nparts; p++) {
    if (!parts[p]) return TBIK_ERR_INVALID;
    if (reinterpret_cast<uintptr_t>(parts[p]) & 1) return TBIK_ERR_ALIGNMENT;
    vec_ok = vec_ok && (reinterpret_cast<uintptr_t>(parts[p]) & 15) == 0;
    a.parts[p] = static_cast<const uint16_t*>(parts[p]);
  }
  a.out = static_cast<uint16_t*>(out);
  a.numel = numel;
  a.bias = static_cast<const uint16_t*>(bias);
  a.ncols = N;
  a.ldo = ldo;
  if (bias) vec_ok = vec_ok && (N & 7) == 0 && (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
  if (ldo) vec_ok = vec_ok && (N & 7) == 0 && (ldo & 7) == 0;
  if (f16) {
    switch (nparts) {
      case 1: return launch_combine<1, true>(a, vec_ok, stream);
      case 2: return launch_combine<2, true>(a, vec_ok, stream);
      case 4: return launch_combine<4, true>(a, vec_ok, stream);
      case 8: return launch_combine<8, true>(a, vec_ok, stream);
      case 16: return launch_combine<16, true>(a, vec_ok, stream);
      default: return launch_combine<32, true>(a, vec_ok, stream);
    }
  }
  switch (nparts) {
    case 1: return launch_combine<1, false>(a, vec_ok, stream);
    case 2: return launch_combine<2, false>(a, vec_ok, stream);
    case 4: return launch_combine<4, false>(a, vec_ok, stream);
    case 8: return launch_combine<8, false>(a, vec_ok, stream);
    case 16: return launch_combine<16, false>(a, vec_ok, stream);
    default: return launch_combine<32, false>(a, vec_ok, stream);
  }
}

int tree_combine_dispatch(const void* const* parts, int nparts, void* out, int64_t numel, bool f16, hipStream_t stream) {
  return tree_combine_bias_dispatch(parts, nparts, out, numel, nullptr, 0, f16, stream, 0);
}

// fp32 partials: a node is one fp32 addition, so only the tree order has to be fixed.  The reference's tree reduce is
// instantiated for float as well (custom_all_reduce.cuh:203-234, custom_all_reduce.cu:118-122).
template <int NP>
__global__ __launch_bounds__(256) void combine_f32_kernel(const CombineArgs a, int64_t npacks) {
  const float* const* parts = reinterpret_cast<const float* const*>(a.parts);
  float* out = reinterpret_cast<float*>(a.out);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t i = first; i < npacks; i += stride) {
    float4 v[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) v[p] = reinterpret_cast<const float4*>(parts[p])[i];
#pragma unroll
    for (int step = 1; step < NP; step <<= 1)
#pragma unroll
      for (int left = 0; left < NP; left += 2 * step) {
        v[left].x += v[left + step].x;
        v[left].y += v[left + step].y;
        v[left].z += v[left + step].z;
        v[left].w += v[left + step].w;
      }
    reinterpret_cast<float4*>(out)[i] = v[0];
  }
  // tail (and everything, when a buffer is not 16-byte aligned: npacks == 0)
  for (int64_t i = npacks * 4 + first; i < a.numel; i += stride) {
    float w[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) w[p] = parts[p][i];
#pragma unroll
    for (int step = 1; step < NP; step <<= 1)
#pragma unroll
      for (int left = 0; left < NP; left += 2 * step) w[left] += w[left + step];
    out[i] = w[0];
  }
}

template <int NP>
static int launch_combine_f32(const CombineArgs& a, bool vec_ok, hipStream_t stream) {
  const int64_t npacks = vec_ok ? a.numel / 4 : 0;
  const int64_t work = npacks > 0 ? npacks : a.numel;
  const int64_t blocks = (work + 255) / 256;
  const unsigned grid = (unsigned)(blocks < 8192 ? blocks : 8192);
  hipLaunchKernelGGL((combine_f32_kernel<NP>), dim3(grid), dim3(256), 0, stream, a, npacks);
  return hip_code(hipGetLastError());
}

int tree_combine_f32_dispatch(const void* const* parts, int nparts, void* out, int64_t numel, hipStream_t stream) {
  if (numel < 0) return TBIK_ERR_INVALID;
  if (nparts < 1 || nparts > 32 || (nparts & (nparts - 1))) return TBIK_ERR_INVALID;
  if (numel == 0) return TBIK_OK;
  if (!parts || !out) return TBIK_ERR_INVALID;
  if (reinterpret_cast<uintptr_t>(out) & 3) return TBIK_ERR_ALIGNMENT;
  CombineArgs a;
  bool vec_ok = (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  for (int p = 0; p < 32; p++) a.parts[p] = nullptr;
  for (int p = 0; p < nparts; p++) {
    if (!parts[p]) return TBIK_ERR_INVALID;
    if (reinterpret_cast<uintptr_t>(parts[p]) & 3) return TBIK_ERR_ALIGNMENT;
    vec_ok = vec_ok && (reinterpret_cast<uintptr_t>(parts[p]) & 15) == 0;
    a.parts[p] = static_cast<const uint16_t*>(parts[p]);
  }
  a.out = static_cast<uint16_t*>(out);
  a.numel = numel;
  a.bias = nullptr;
  a.ncols = 0;
  a.ldo = 0;
  switch (nparts) {
    case 1: return launch_combine_f32<1>(a, vec_ok, stream);
    case 2: return launch_combine_f32<2>(a, vec_ok, stream);
    case 4: return launch_combine_f32<4>(a, vec_ok, stream);
    case 8: return launch_combine_f32<8>(a, vec_ok, stream);
    case 16: return launch_combine_f32<16>(a, vec_ok, stream);
    default: return launch_combine_f32<32>(a, vec_ok, stream);
  }
}

}  // namespace tbik
