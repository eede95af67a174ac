// Argument blocks and entry points of the large-M GEMM kernels, shared by the kernels' own files and by the
// dispatcher in gemm_tiled.hip.
#pragma once
#include "common.h"

namespace tbik {

// gemm_tree_wide.hip: tree-ordered bf16 / fp16 GEMM, 128x256 tiles
struct WideArgs {
  const uint16_t* X;   // [M,K], row stride ldx
  const uint16_t* W;   // [N,K], row stride ldw
  uint16_t* C;         // [M,N], row stride ldc
  const uint16_t* bias;
  u32x4* ws;           // parked tree levels: [level][shard * tile][wave][chunk 0..7][lane]
  int64_t ldx, ldw, ldc;
  int M, N, K;
  int T, flb, lb;
  int vec_store;
  int64_t k_shard, c_shard;  // K split over gridDim.y shards: operand column offset and partial-output offset per shard
};
// bytes of parked tree levels: one slab of 16 B per lane per level beyond those the kernel keeps in registers (1 for
// gemm_tree_wide.hip, 2 for gemm_tree_wide_deep.hip; both kernels use the same tile grid and the same slab layout)
size_t wide_workspace_bytes(int M, int N, int lb, int split, int levels_in_registers);
int gemm_tree_wide_launch(const WideArgs& a, int leaf_k, bool f16, int split, hipStream_t stream);
// gemm_tree_wide_deep.hip: the same tile and bits for leaves of 256 with two binary levels in registers (a.lb >= 2 uses
// both); takes the same arguments
int gemm_tree_deep_launch(const WideArgs& a, int split, hipStream_t stream);
// Two problems in ONE launch of either kernel (column regions of one GEMM, each with a K split of its own): the
// work-groups of `first` come first in the grid (give it the longer shards, so that the short work-groups of `second`
// fill the CUs that finish early), then those of `second`; every work-group computes what it would compute in a launch
// of its problem alone.
struct WidePair {
  WideArgs first, second;
  int split_first, split_second;
};
template <bool PAIR> struct WideKernelArgs { using type = WideArgs; };
template <> struct WideKernelArgs<true> { using type = WidePair; };
int gemm_tree_wide_pair_launch(const WidePair& a, int leaf_k, bool f16, hipStream_t stream);
int gemm_tree_deep_pair_launch(const WidePair& a, hipStream_t stream);

// gemm_tree_quad.hip: tree-ordered bf16 GEMM with leaves of 256 on 128x128 tiles (one wave per SIMD, the tree of a shard
// in registers: a.lb <= 1, a.ws unused); grid.y = split as for the kernels above
int gemm_tree_quad_launch(const WideArgs& a, int split, hipStream_t stream);

// gemm_single_acc_quad.hip: single-accumulator bf16 GEMM, one wave per SIMD
struct QuadArgs {
  const uint16_t* X;   // [M,K], row stride ldx
  const uint16_t* W;   // [N,K], row stride ldw
  uint16_t* C;         // [M,N], row stride ldc
  const uint16_t* bias;
  int64_t ldx, ldw, ldc;
  int M, N, K;
  int vec_store;
  int row_step = 0;    // rows a tile of gemm_single_acc_quad_kernel owns (0 = all 128; 64, 32 or 16: see the kernel)
};
int gemm_single_acc_quad_launch(const QuadArgs& a, hipStream_t stream);
int gemm_single_acc_slab_launch(const QuadArgs& a, hipStream_t stream);  // at most 128 rows; TBIK_ERR_UNSUPPORTED: use another kernel
int gemm_single_acc_balanced_launch(const QuadArgs& a, hipStream_t stream);  // any row count: tile width from a cost model
// gemm_single_acc_256.hip: the same GEMM on tiles of 256 or 192 rows by 256 or 192 columns, for grids of more than one
// round; K % 64 == 0
int gemm_single_acc_256_launch(const QuadArgs& a, int tile_rows, int tile_cols, hipStream_t stream);

// gemm_single_acc_stream.hip: single-accumulator 16-bit GEMM for at most 64 rows, weights streamed from global memory
struct StreamArgs {
  const uint16_t* X;   // [M,K], row stride ldx
  const uint16_t* W;   // [N,K], row stride ldw
  uint16_t* C;         // [M,N], row stride ldc
  const uint16_t* bias;
  int64_t ldx, ldw, ldc;
  int M, N, K;
  int vec_store;
  const uint16_t* W2 = nullptr;  // gated form only: the second weight matrix [N,K] (the `up` half of a merged projection)
};
int gemm_single_acc_stream_launch(const StreamArgs& a, bool f16, hipStream_t stream);
// C[M,N] = silu(X W^T) * (X W2^T), both products rounded to the element type first (the bits of the mm followed by the
// activation kernel), for the row counts of the windowed kernel; TBIK_ERR_UNSUPPORTED otherwise (nothing launched)
int gemm_single_acc_stream_gated_launch(const StreamArgs& a, hipStream_t stream);
// the same product with X = RMSNorm(a.X [+ res]) * w formed while the activations are staged (bf16, a few rows);
// res_out receives the rounded sum a.X + res when res is given; TBIK_ERR_UNSUPPORTED: run the two launches
struct StreamNormArgs {
  const uint16_t* res = nullptr;
  const uint16_t* w = nullptr;
  uint16_t* res_out = nullptr;
  int64_t ldr = 0, ldro = 0;
  float eps = 0.f;
};
int gemm_single_acc_stream_norm_launch(const StreamArgs& a, const StreamNormArgs& nrm, hipStream_t stream);

// gemm_tree_strip.hip: tree-ordered 16-bit GEMM for at most 16 rows, K cut over the waves of a work-group
struct StripArgs {
  const uint16_t* X;   // [M,K], row stride ldx
  const uint16_t* W;   // [N,K], row stride ldw
  uint16_t* C;         // [M,N], row stride ldc
  const uint16_t* bias;
  int64_t ldx, ldw, ldc;
  int M, N, K;
  int flb, lb;         // K = flb * leaf_k * 2^lb
  int vec_store;
  const uint16_t* X2 = nullptr;  // gated form only: X = gate rows, X2 = up rows (same row stride)
};
int gemm_tree_strip_waves(int M, int N, int K, int lb);  // waves per strip, or 0: use another kernel
int gemm_tree_strip_launch(const StripArgs& a, int leaf_k, int waves, bool f16, hipStream_t stream);
// the same kernel with the activations silu(a.X) * a.X2 (gate and up rows, [M,K] each, row stride a.ldx) formed while
// the first weights are in flight (bf16, at most 4 rows); waves = 0: run the two launches
int gemm_tree_strip_gated_waves(int M, int N, int K, int lb);
int gemm_tree_strip_gated_launch(const StripArgs& a, int leaf_k, int waves, hipStream_t stream);

// tree_combine.hip
// ldo != 0: `out` is a [numel / N, N] matrix with row stride ldo (the partials stay contiguous)
int tree_combine_bias_dispatch(const void* const* parts, int nparts, void* out, int64_t numel, const void* bias, int N,
                               bool f16, hipStream_t stream, int64_t ldo = 0);

// the shard combine with the (add-)RMSNorm of the combined rows behind it in the same launch: out = normalised rows,
// res_out = combined + residual (with res), sum_out (optional) = the combined rows themselves
int tree_combine_rmsnorm_dispatch(const void* const* parts, int nparts, int64_t rows, int hidden, const void* bias,
                                  const void* res, int64_t ldr, const void* w, float eps, void* out, int64_t ldo,
                                  void* res_out, int64_t ldro, void* sum_out, int64_t lds, bool f16, hipStream_t stream);

// What follows a tree matmul whose K split ends in a shard combine, when the caller wants the (add-)RMSNorm of the result
// in that combine's launch: the matmul's C / ldc arguments then name the NORMALISED output.
struct NormEpilogue {
  const void* res;   // optional residual [M, ldr]
  int64_t ldr;
  const void* w;     // optional norm weight [N]
  float eps;
  void* res_out;     // result + residual [M, ldro] (with res)
  int64_t ldro;
};

}  // namespace tbik
