// extern "C" surface of libtbik_hip.so (declared in include/tbik_hip.h): argument checks live in the
// dispatchers next to each kernel, this file only binds names.
#include "common.h"

namespace tbik {
int gemm_dispatch(bool tree, bool f16, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                  int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, void* ws, size_t ws_bytes,
                  hipStream_t stream);
size_t gemm_workspace_bytes(int M, int N, int K, int leaf_k, bool f16, bool rowmajor_b = false);
int gemm_plan_info(int M, int N, int K, int leaf_k, bool f16, bool rowmajor_b, int out[5]);
int tree_combine_dispatch(const void* const* parts, int nparts, void* out, int64_t numel, bool f16, hipStream_t stream);
int tree_combine_f32_dispatch(const void* const* parts, int nparts, void* out, int64_t numel, hipStream_t stream);
int rmsnorm_dispatch(const void* x, int64_t ldx, const void* res, int64_t ldr, const void* w, void* out, int64_t ldo,
                     void* res_out, int64_t ldro, int64_t rows, int hidden, float eps, bool f16, hipStream_t stream);
size_t lsm_workspace_bytes(int64_t rows, int64_t cols);
int log_softmax_dispatch(const void* x, int64_t ldx, int in_dtype, void* out, int64_t ldo, int out_dtype, int64_t rows,
                         int64_t cols, void* ws, size_t ws_bytes, int write_softmax, hipStream_t stream);
int attention_dispatch(const void* q, const void* k_cache, const void* vt_cache, void* out, const int* q_start,
                       const int* q_len, const int* ctx_len, int batch, int max_q_len, int q_heads, int kv_heads,
                       int head_dim, int max_len, float scale, hipStream_t stream);
int argmax_dispatch(const void* x, int64_t ld, void* out, int64_t rows, int cols, void* history, int64_t history_ld,
                    void* count, void* positions, void* ctx_len, hipStream_t stream);
int mean_dispatch(const void* x, void* out, int64_t outer, int64_t n, int64_t inner, int dtype_code, hipStream_t stream);
int gemm_f32_dispatch(bool tree, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                      int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, hipStream_t stream);
int qk_norm_rope_cache_dispatch(const void* qkv, int64_t ld, const void* q_weight, const void* k_weight,
                                const float* inv_freq, const int64_t* positions, const int64_t* seq_of_token, void* q_out,
                                void* k_cache, void* vt_cache, int64_t tokens, int q_heads, int kv_heads, int head_dim,
                                int max_len, int batch, float eps, hipStream_t stream);
int silu_mul_dispatch(const void* gate_up, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int inter, bool f16,
                      hipStream_t stream);
int rmsnorm_gemm_dispatch(const void* x, int64_t ldx, const void* res, int64_t ldr, const void* norm_w, float eps,
                          void* res_out, int64_t ldro, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc,
                          int M, int N, int K, const void* bias, hipStream_t stream);
int attention_decode_qkv_dispatch(const void* qkv, int64_t ld, const void* q_weight, const void* k_weight, const float* inv_freq,
                                  void* k_cache, void* vt_cache, void* out, const int* ctx_len, int batch, int q_heads,
                                  int kv_heads, int head_dim, int max_len, float scale, float eps, hipStream_t stream);
int gemm_silu_mul_dispatch(const void* x, int64_t ldx, const void* W, int64_t ldw, void* out, int64_t ldo, int M, int inter, int K,
                           hipStream_t stream);
int gemm_tree_rmsnorm_dispatch(bool f16, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, int M, int N,
                               int K, int leaf_k, const void* bias, const void* res, int64_t ldr, const void* norm_w, float eps,
                               void* res_out, int64_t ldro, void* out, int64_t ldo, void* ws, size_t ws_bytes,
                               hipStream_t stream);
int tree_combine_rmsnorm_dispatch(const void* const* parts, int nparts, int64_t rows, int hidden, const void* bias,
                                  const void* res, int64_t ldr, const void* w, float eps, void* out, int64_t ldo,
                                  void* res_out, int64_t ldro, void* sum_out, int64_t lds, bool f16, hipStream_t stream);
int gemm_tree_gated_dispatch(const void* gate, const void* up, int64_t ld, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                             int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, hipStream_t stream);
}  // namespace tbik

extern "C" {

int tbik_abi_version(void) { return 17; }

const char* tbik_error_string(int code) {
  switch (code) {
    case TBIK_OK: return "ok";
    case TBIK_ERR_INVALID: return "invalid argument (shape, null pointer, or K not a whole number of leaves)";
    case TBIK_ERR_ALIGNMENT: return "pointer or leading dimension not aligned for 16-byte accesses";
    case TBIK_ERR_UNSUPPORTED: return "layout, dtype or tree depth not supported by this build";
    case TBIK_ERR_WORKSPACE: return "workspace missing or too small";
    case TBIK_ERR_SCRATCH_LIMIT: return "the problem needs more scratch than the library's fixed array (TBIK_STATIC_SCRATCH_BYTES): use the entry point that takes a workspace";
    default: return code >= TBIK_ERR_HIP_BASE ? hipGetErrorString((hipError_t)(code - TBIK_ERR_HIP_BASE)) : "unknown";
  }
}

int tbik_tree_params(int K, int leaf_k, int* T, int* flb, int* level_k) {
  if (K <= 0 || leaf_k <= 0 || K % leaf_k != 0 || !T || !flb || !level_k) return TBIK_ERR_INVALID;
  int t = K / leaf_k, f = t, l = 1;
  while (f > 2 && (f & 1) == 0) {
    f >>= 1;
    l++;
  }
  *T = t;
  *flb = f;
  *level_k = l;
  return TBIK_OK;
}

size_t tbik_gemm_workspace_bytes(int M, int N, int K, int leaf_k) { return tbik::gemm_workspace_bytes(M, N, K, leaf_k, false); }
size_t tbik_gemm_f16_workspace_bytes(int M, int N, int K, int leaf_k) { return tbik::gemm_workspace_bytes(M, N, K, leaf_k, true); }
size_t tbik_gemm_workspace_bytes_rowmajor_b(int M, int N, int K, int leaf_k, int f16) {
  return tbik::gemm_workspace_bytes(M, N, K, leaf_k, f16 != 0, true);
}
int tbik_gemm_plan_info(int M, int N, int K, int leaf_k, int f16, int rowmajor_b, int* out5) {
  return tbik::gemm_plan_info(M, N, K, leaf_k, f16 != 0, rowmajor_b != 0, out5);
}

int tbik_gemm_bf16(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc, int M,
                   int N, int K, int leaf_k, const void* bias_or_null, void* workspace, size_t workspace_bytes,
                   tbik_stream_t stream) {
  return tbik::gemm_dispatch(true, false, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, leaf_k, bias_or_null, workspace,
                             workspace_bytes, static_cast<hipStream_t>(stream));
}

int tbik_tree_combine_bf16(const void* const* parts, int nparts, void* out, int64_t numel, tbik_stream_t stream) {
  return tbik::tree_combine_dispatch(parts, nparts, out, numel, false, static_cast<hipStream_t>(stream));
}

int tbik_gemm_f16(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc, int M,
                  int N, int K, int leaf_k, const void* bias_or_null, void* workspace, size_t workspace_bytes,
                  tbik_stream_t stream) {
  return tbik::gemm_dispatch(true, true, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, leaf_k, bias_or_null, workspace,
                             workspace_bytes, static_cast<hipStream_t>(stream));
}

int tbik_tree_combine_f16(const void* const* parts, int nparts, void* out, int64_t numel, tbik_stream_t stream) {
  return tbik::tree_combine_dispatch(parts, nparts, out, numel, true, static_cast<hipStream_t>(stream));
}

int tbik_tree_combine_f32(const void* const* parts, int nparts, void* out, int64_t numel, tbik_stream_t stream) {
  return tbik::tree_combine_f32_dispatch(parts, nparts, out, numel, static_cast<hipStream_t>(stream));
}

int bi_gemm_f16(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc, int M,
                int N, int K, const void* bias_or_null, tbik_stream_t stream) {
  return tbik::gemm_dispatch(false, true, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, 0, bias_or_null, nullptr, 0,
                             static_cast<hipStream_t>(stream));
}

int bi_gemm_bf16(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc, int M,
                 int N, int K, const void* bias_or_null, tbik_stream_t stream) {
  return tbik::gemm_dispatch(false, false, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, 0, bias_or_null, nullptr, 0,
                             static_cast<hipStream_t>(stream));
}

int bi_rmsnorm_gemm_bf16(const void* x, int64_t ldx, const void* residual_or_null, int64_t ldr, const void* norm_weight_or_null,
                         float eps, void* residual_out_or_null, int64_t ldro, const void* B, int64_t ldb_k, int64_t ldb_n,
                         void* C, int64_t ldc, int M, int N, int K, const void* bias_or_null, tbik_stream_t stream) {
  return tbik::rmsnorm_gemm_dispatch(x, ldx, residual_or_null, ldr, norm_weight_or_null, eps, residual_out_or_null, ldro, B,
                                     ldb_k, ldb_n, C, ldc, M, N, K, bias_or_null, static_cast<hipStream_t>(stream));
}

int tbik_gemm_silu_mul_bf16(const void* gate, const void* up, int64_t ld, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                            int64_t ldc, int M, int N, int K, int leaf_k, const void* bias_or_null, tbik_stream_t stream) {
  return tbik::gemm_tree_gated_dispatch(gate, up, ld, B, ldb_k, ldb_n, C, ldc, M, N, K, leaf_k, bias_or_null,
                                        static_cast<hipStream_t>(stream));
}

int bi_gemm_silu_mul_bf16(const void* x, int64_t ldx, const void* W, int64_t ldw, void* out, int64_t ldo, int M, int inter, int K,
                          tbik_stream_t stream) {
  return tbik::gemm_silu_mul_dispatch(x, ldx, W, ldw, out, ldo, M, inter, K, static_cast<hipStream_t>(stream));
}

int tbik_gemm_rmsnorm_bf16(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, int M, int N, int K,
                           int leaf_k, const void* bias_or_null, const void* residual_or_null, int64_t ldr,
                           const void* norm_weight_or_null, float eps, void* residual_out_or_null, int64_t ldro, void* out,
                           int64_t ldo, void* workspace, size_t workspace_bytes, tbik_stream_t stream) {
  return tbik::gemm_tree_rmsnorm_dispatch(false, A, lda, B, ldb_k, ldb_n, M, N, K, leaf_k, bias_or_null, residual_or_null, ldr,
                                          norm_weight_or_null, eps, residual_out_or_null, ldro, out, ldo, workspace,
                                          workspace_bytes, static_cast<hipStream_t>(stream));
}

int tbik_tree_combine_rmsnorm_bf16(const void* const* parts, int nparts, int64_t rows, int hidden, const void* bias_or_null,
                                   const void* residual_or_null, int64_t ldr, const void* norm_weight_or_null, float eps,
                                   void* residual_out_or_null, int64_t ldro, void* out, int64_t ldo, tbik_stream_t stream) {
  return tbik::tree_combine_rmsnorm_dispatch(parts, nparts, rows, hidden, bias_or_null, residual_or_null, ldr,
                                             norm_weight_or_null, eps, out, ldo, residual_out_or_null, ldro, nullptr, 0, false,
                                             static_cast<hipStream_t>(stream));
}

int bi_rmsnorm_bf16(const void* x, int64_t ldx, const void* residual_or_null, int64_t ldr, const void* weight_or_null,
                    void* out, int64_t ldo, void* residual_out_or_null, int64_t ldro, int64_t rows, int hidden, float eps,
                    tbik_stream_t stream) {
  return tbik::rmsnorm_dispatch(x, ldx, residual_or_null, ldr, weight_or_null, out, ldo, residual_out_or_null, ldro, rows,
                                hidden, eps, false, static_cast<hipStream_t>(stream));
}

int bi_rmsnorm_f16(const void* x, int64_t ldx, const void* residual_or_null, int64_t ldr, const void* weight_or_null,
                   void* out, int64_t ldo, void* residual_out_or_null, int64_t ldro, int64_t rows, int hidden, float eps,
                   tbik_stream_t stream) {
  return tbik::rmsnorm_dispatch(x, ldx, residual_or_null, ldr, weight_or_null, out, ldo, residual_out_or_null, ldro, rows,
                                hidden, eps, true, static_cast<hipStream_t>(stream));
}

size_t bi_log_softmax_workspace_bytes(int64_t rows, int64_t cols) { return tbik::lsm_workspace_bytes(rows, cols); }

int bi_log_softmax_f32(const void* x, int64_t ldx, void* out, int64_t ldo, int64_t rows, int64_t cols, void* workspace,
                       size_t workspace_bytes, int write_softmax, tbik_stream_t stream) {
  return tbik::log_softmax_dispatch(x, ldx, 0, out, ldo, 0, rows, cols, workspace, workspace_bytes, write_softmax,
                                    static_cast<hipStream_t>(stream));
}

int bi_log_softmax(const void* x, int64_t ldx, int in_dtype_code, void* out, int64_t ldo, int out_dtype_code, int64_t rows,
                   int64_t cols, void* workspace, size_t workspace_bytes, int write_softmax, tbik_stream_t stream) {
  return tbik::log_softmax_dispatch(x, ldx, in_dtype_code, out, ldo, out_dtype_code, rows, cols, workspace, workspace_bytes,
                                    write_softmax, static_cast<hipStream_t>(stream));
}

int bi_mean_dim(const void* x, void* out, int64_t outer, int64_t n, int64_t inner, int dtype_code, tbik_stream_t stream) {
  return tbik::mean_dispatch(x, out, outer, n, inner, dtype_code, static_cast<hipStream_t>(stream));
}

int bi_attention_bf16(const void* q, const void* k_cache, const void* vt_cache, void* out, const int32_t* q_start,
                      const int32_t* q_len, const int32_t* ctx_len, int batch, int max_q_len, int q_heads, int kv_heads,
                      int head_dim, int max_len, float scale, tbik_stream_t stream) {
  return tbik::attention_dispatch(q, k_cache, vt_cache, out, q_start, q_len, ctx_len, batch, max_q_len, q_heads, kv_heads,
                                  head_dim, max_len, scale, static_cast<hipStream_t>(stream));
}

int tbik_gemm_f32(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc, int M,
                  int N, int K, int leaf_k, const void* bias_or_null, tbik_stream_t stream) {
  return tbik::gemm_f32_dispatch(true, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, leaf_k, bias_or_null,
                                 static_cast<hipStream_t>(stream));
}

int bi_gemm_f32(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C, int64_t ldc, int M,
                int N, int K, const void* bias_or_null, tbik_stream_t stream) {
  return tbik::gemm_f32_dispatch(false, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, 0, bias_or_null,
                                 static_cast<hipStream_t>(stream));
}

int bi_silu_mul_bf16(const void* gate_up, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int inter,
                     tbik_stream_t stream) {
  return tbik::silu_mul_dispatch(gate_up, ld_in, out, ld_out, rows, inter, false, static_cast<hipStream_t>(stream));
}

int bi_silu_mul_f16(const void* gate_up, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int inter,
                    tbik_stream_t stream) {
  return tbik::silu_mul_dispatch(gate_up, ld_in, out, ld_out, rows, inter, true, static_cast<hipStream_t>(stream));
}

int bi_qk_norm_rope_cache_bf16(const void* qkv, int64_t ld, const void* q_weight, const void* k_weight,
                                const float* inv_freq, const int64_t* positions, const int64_t* seq_of_token, void* q_out,
                                void* k_cache, void* vt_cache, int64_t tokens, int q_heads, int kv_heads, int head_dim,
                                int max_len, int batch, float eps, tbik_stream_t stream) {
  return tbik::qk_norm_rope_cache_dispatch(qkv, ld, q_weight, k_weight, inv_freq, positions, seq_of_token, q_out, k_cache,
                                           vt_cache, tokens, q_heads, kv_heads, head_dim, max_len, batch, eps,
                                           static_cast<hipStream_t>(stream));
}

int bi_attention_decode_qkv_bf16(const void* qkv, int64_t ld, const void* q_weight, const void* k_weight, const float* inv_freq,
                                 void* k_cache, void* vt_cache, void* out, const int32_t* ctx_len, int batch, int q_heads,
                                 int kv_heads, int head_dim, int max_len, float scale, float eps, tbik_stream_t stream) {
  return tbik::attention_decode_qkv_dispatch(qkv, ld, q_weight, k_weight, inv_freq, k_cache, vt_cache, out, ctx_len, batch,
                                             q_heads, kv_heads, head_dim, max_len, scale, eps, static_cast<hipStream_t>(stream));
}

int bi_argmax_bf16(const void* x, int64_t ld, void* out, int64_t rows, int cols, tbik_stream_t stream) {
  return tbik::argmax_dispatch(x, ld, out, rows, cols, nullptr, 0, nullptr, nullptr, nullptr, static_cast<hipStream_t>(stream));
}

int bi_argmax_advance_bf16(const void* x, int64_t ld, void* next_token, int64_t rows, int cols, void* history,
                           int64_t history_ld, void* count, void* positions, void* ctx_len, tbik_stream_t stream) {
  return tbik::argmax_dispatch(x, ld, next_token, rows, cols, history, history_ld, count, positions, ctx_len,
                               static_cast<hipStream_t>(stream));
}

}  // extern "C"
