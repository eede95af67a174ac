// Shard combine: out[i] = adjacent-pair binary tree over up to 32 bf16 (or fp16) partials, every node rounded to
// the element type.  This is the arithmetic of the reference's cross-GPU tree all-reduce
// (src/tbik/tree_based_all_reduce.py:32-37; packed_tree_reduce,
// mini_allreduce/tbik_kernel/csrc/allreduce/custom_all_reduce.cuh:203-234) applied to partials that
// already sit in one GPU's memory.  HBM bound: (nparts + 1) * numel * 2 bytes.
#include "common.h"
#include "rmsnorm_row.h"

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

// The tree over the NP partial packs of one 16-byte pack (8 elements), and the bias added to it: one body for every
// kernel that combines shards, so they all give the same bits.
template <int NP, bool F16>
__device__ __forceinline__ uint4 combine_pack(const uint4 (&in)[NP]) {
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
  return o;
}

template <bool F16>
__device__ __forceinline__ uint4 add_pack(const uint4& o, const uint4& bq) {
  return make_uint4(Num16<F16>::add(o.x, bq.x), Num16<F16>::add(o.y, bq.y), Num16<F16>::add(o.z, bq.z), Num16<F16>::add(o.w, bq.w));
}

// One thread per 16-byte pack (8 bf16); grid-stride so any numel fits one launch.
template <int NP, bool F16>
__global__ __launch_bounds__(256) void combine_vec_kernel(const CombineArgs a, int64_t npacks) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < npacks; i += stride) {
    uint4 in[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) in[p] = reinterpret_cast<const uint4*>(a.parts[p])[i];
    uint4 o = combine_pack<NP, F16>(in);
    // ncols % 8 == 0 on this path: the pack stays inside one row
    if (a.bias) o = add_pack<F16>(o, *reinterpret_cast<const uint4*>(a.bias + (i * 8) % a.ncols));
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

// ------------------------------------------------------------------------------------------------
// Shard combine followed by the (add-)RMSNorm of the combined rows, in one launch: the row's packs are formed exactly
// as combine_vec_kernel forms them (tree over the partials, then the bias) and handed, without a trip through memory,
// to the row function of the stand-alone RMSNorm (rmsnorm_row.h) in the lane layout that function expects.
// Same bits as the two launches; a decode-sized batch saves a kernel per row-split layer.
// ------------------------------------------------------------------------------------------------
struct CombineNormArgs {
  const uint16_t* parts[32];  // [rows, hidden] each, contiguous
  const uint16_t* bias;       // optional [hidden]
  const uint16_t* res;        // optional residual [rows, ldr]
  const uint16_t* w;          // optional norm weight [hidden]
  uint16_t* out;              // normalised rows [rows, ldo]
  uint16_t* res_out;          // combined + residual [rows, ldro] (with res)
  uint16_t* sum_out;          // optional: the combined rows themselves [rows, lds]
  int64_t ldr, ldo, ldro, lds;
  int64_t rows;
  int hidden;
  float eps;
};

// One work-group per row, CPL wavefronts: wave w forms the chunks lane + 64 w of the row (all its partial loads in
// flight at once) and leaves them in LDS; wave 0, which asked for the residual and the weights first, then takes the
// whole row in the lane layout of the row function (lane l: chunks l, l + 64, ...) and finishes it.
template <int NP, int CPL, bool F16>
__global__ __launch_bounds__(64 * CPL) void combine_rmsnorm_kernel(const CombineNormArgs a) {
  __shared__ uint4 xs[64 * CPL];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t row = blockIdx.x;
  const int nchunks = a.hidden >> 3;
  RmsnormRow<CPL, F16> r;
  r.has_res = a.res != nullptr;
  r.has_w = a.w != nullptr;
  if (wave == 0) {
    const uint4* wr = reinterpret_cast<const uint4*>(a.w);
    const uint4* rr = a.res ? reinterpret_cast<const uint4*>(a.res + row * a.ldr) : nullptr;
#pragma unroll
    for (int i = 0; i < CPL; i++) {
      const int c = lane + 64 * i;
      if (c < nchunks) {
        if (wr) r.wq[i] = wr[c];
        if (rr) r.rq[i] = rr[c];
      }
    }
  }
  const int c = lane + 64 * wave;
  if (c < nchunks) {
    uint4 in[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) in[p] = reinterpret_cast<const uint4*>(a.parts[p] + row * a.hidden)[c];
    uint4 o = combine_pack<NP, F16>(in);
    if (a.bias) o = add_pack<F16>(o, reinterpret_cast<const uint4*>(a.bias)[c]);
    if (a.sum_out) reinterpret_cast<uint4*>(a.sum_out + row * a.lds)[c] = o;
    xs[c] = o;
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int i = 0; i < CPL; i++) {
    const int ci = lane + 64 * i;
    if (ci < nchunks) r.xq[i] = xs[ci];
  }
  uint4* orow = reinterpret_cast<uint4*>(a.out + row * a.ldo);
  r.finish(a.res_out ? a.res_out + row * a.ldro : nullptr, a.hidden, a.eps, lane, [&](int cc, const uint4& o) { orow[cc] = o; });
}

template <int NP, bool F16>
static void launch_combine_rmsnorm(const CombineNormArgs& a, dim3 grid, hipStream_t stream) {
  const int cpl = (a.hidden + 511) / 512;  // a function of the row length only
  if (cpl <= 2) hipLaunchKernelGGL((combine_rmsnorm_kernel<NP, 2, F16>), grid, dim3(128), 0, stream, a);
  else if (cpl <= 8) hipLaunchKernelGGL((combine_rmsnorm_kernel<NP, 8, F16>), grid, dim3(512), 0, stream, a);
  else hipLaunchKernelGGL((combine_rmsnorm_kernel<NP, 16, F16>), grid, dim3(1024), 0, stream, a);
}

int tree_combine_rmsnorm_dispatch(const void* const* parts, int nparts, int64_t rows, int hidden, const void* bias,
                                  const void* res, int64_t ldr, const void* w, float eps, void* out, int64_t ldo,
                                  void* res_out, int64_t ldro, void* sum_out, int64_t lds, bool f16, hipStream_t stream) {
  if (rows < 0 || hidden <= 0) return TBIK_ERR_INVALID;
  if (nparts < 2 || nparts > 32 || (nparts & (nparts - 1))) return TBIK_ERR_INVALID;
  if (rows == 0) return TBIK_OK;
  if (!parts || !out || (res && !res_out)) return TBIK_ERR_INVALID;
  if (hidden & 7) return TBIK_ERR_ALIGNMENT;
  if (hidden > 16 * 512) return TBIK_ERR_UNSUPPORTED;
  auto bad = [](const void* p, int64_t ld) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0 || (ld & 7) != 0; };
  if (bad(out, ldo) || (res && (bad(res, ldr) || bad(res_out, ldro))) || (w && bad(w, 8)) || (bias && bad(bias, 8)) ||
      (sum_out && bad(sum_out, lds)))
    return TBIK_ERR_ALIGNMENT;
  if (ldo < hidden || (res && (ldr < hidden || ldro < hidden)) || (sum_out && lds < hidden)) return TBIK_ERR_INVALID;
  CombineNormArgs a;
  for (int p = 0; p < 32; p++) a.parts[p] = nullptr;
  for (int p = 0; p < nparts; p++) {
    if (!parts[p]) return TBIK_ERR_INVALID;
    if (reinterpret_cast<uintptr_t>(parts[p]) & 15) return TBIK_ERR_ALIGNMENT;
    a.parts[p] = static_cast<const uint16_t*>(parts[p]);
  }
  a.bias = static_cast<const uint16_t*>(bias);
  a.res = static_cast<const uint16_t*>(res);
  a.w = static_cast<const uint16_t*>(w);
  a.out = static_cast<uint16_t*>(out);
  a.res_out = static_cast<uint16_t*>(res ? res_out : nullptr);
  a.sum_out = static_cast<uint16_t*>(sum_out);
  a.ldr = ldr;
  a.ldo = ldo;
  a.ldro = ldro;
  a.lds = lds;
  a.rows = rows;
  a.hidden = hidden;
  a.eps = eps;
  if (rows > 0x7fffffff) return TBIK_ERR_INVALID;
  const dim3 grid((unsigned)rows);
  if (f16) {
    switch (nparts) {
      case 2: launch_combine_rmsnorm<2, true>(a, grid, stream); break;
      case 4: launch_combine_rmsnorm<4, true>(a, grid, stream); break;
      case 8: launch_combine_rmsnorm<8, true>(a, grid, stream); break;
      case 16: launch_combine_rmsnorm<16, true>(a, grid, stream); break;
      default: launch_combine_rmsnorm<32, true>(a, grid, stream); break;
    }
  } else {
    switch (nparts) {
      case 2: launch_combine_rmsnorm<2, false>(a, grid, stream); break;
      case 4: launch_combine_rmsnorm<4, false>(a, grid, stream); break;
      case 8: launch_combine_rmsnorm<8, false>(a, grid, stream); break;
      case 16: launch_combine_rmsnorm<16, false>(a, grid, stream); break;
      default: launch_combine_rmsnorm<32, false>(a, grid, stream); break;
    }
  }
  return hip_code(hipGetLastError());
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
