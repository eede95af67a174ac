/*
 * libtbik_hip.so -- C ABI of the MI355X (gfx950) tree-based invariant kernels.
 *
 * Every entry point
 *   - takes plain device pointers, sizes and element strides (no torch types),
 *   - enqueues its kernels on the caller's `stream` (a hipStream_t; NULL = the default stream),
 *   - allocates nothing, synchronises nothing and is re-entrant; the only state it keeps is a once-per-device
 *     flag per kernel that remembers that the kernel's dynamic-LDS limit has been raised on that device,
 *   - validates shapes / alignment on the host BEFORE launching and returns a TBIK_* code
 *     (0 = success); codes >= TBIK_ERR_HIP_BASE are TBIK_ERR_HIP_BASE + hipError_t.
 *
 * Each declaration cites the interface of the reference (nanomaoli/llm_reproducibility) that it
 * replaces; paths are relative to the reference checkout.
 */
#ifndef TBIK_HIP_H
#define TBIK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TBIK_OK               0
#define TBIK_ERR_INVALID      1   /* bad shape / null pointer / K not a whole number of leaves      */
#define TBIK_ERR_ALIGNMENT    2   /* pointer or leading dimension not aligned for 16-byte accesses  */
#define TBIK_ERR_UNSUPPORTED  3   /* layout or tree depth this build has no kernel for              */
#define TBIK_ERR_WORKSPACE    4   /* workspace missing or too small                                 */
#define TBIK_ERR_SCRATCH_LIMIT 5  /* the problem needs more than TBIK_STATIC_SCRATCH_BYTES of scratch */
#define TBIK_ERR_HIP_BASE     1000

typedef void* tbik_stream_t;  /* hipStream_t */

/* ABI version of this header (bumped when a signature changes). */
int tbik_abi_version(void);

/* Static text for a TBIK_* code. */
const char* tbik_error_string(int code);

/*
 * Tree parameters of a K extent: T = K / leaf_k leaves, FLB = T with factors of two removed while
 * even and > 2, LEVEL_K = halvings + 1.
 * Replaces: the host arithmetic of matmul_tp_persistent, src/tbik/tree_based_matmul.py:242-249.
 */
int tbik_tree_params(int K, int leaf_k, int* T, int* flb, int* level_k);

/*
 * C[M,N] (bf16) = tree-ordered A[M,K] x B[K,N] (+ bias[N], added in bf16 after the tree).
 * K is cut into leaves of leaf_k (256 = the reference's bf16 BLOCK_K; 128 is accepted for layers
 * whose shards are not a multiple of 256).  Each leaf is accumulated in fp32 by a fixed chain of
 * 16x16x32 bf16 MFMAs and rounded once to bf16; leaves are merged level 0 left-to-right over FLB
 * leaves and then by an adjacent-pair binary tree, every node rounded to bf16.  The value of
 * C[m,n] depends only on row m of A and column n of B -- not on M, N, the tile configuration or
 * the launch.
 *   A: element (m,k) at A[m*lda + k]                       (K contiguous)
 *   B: element (k,n) at B[k*ldb_k + n*ldb_n], as the reference passes B's strides to its kernel
 *      (src/tbik/tree_based_matmul.py:259-264).  ldb_k == 1 (the nn.Linear weight [N,K], i.e. weight.t()) is the
 *      native layout of every kernel; ldb_n == 1 (row-major [K,N], what simple_matmul.py:11-14 hands over) is
 *      consumed in place by the tiled kernels, which transpose 8x8 blocks in registers on the way to LDS -- same
 *      MFMA chain, same bits, no copy (the large-M pipelines are built for [N,K] only: measured on MI355X,
 *      [M,12288] x [12288,4096] row-major takes 60 / 762 us at M = 128 / 2048 against 32 / 200 us for the [N,K]
 *      form, so a caller with many rows should hand over [N,K]; the Python wrappers repack from 1024
 *      rows on).  The contiguous dimension's partner stride must be a multiple of 8 elements;
 *      neither stride equal to 1 returns TBIK_ERR_UNSUPPORTED.
 *      For ldb_n == 1 the workspace size is tbik_gemm_workspace_bytes_rowmajor_b(M,N,K,leaf_k,f16).
 *   C: element (m,n) at C[m*ldc + n]
 *   workspace: at least tbik_gemm_workspace_bytes(M,N,K,leaf_k) bytes, 16-byte aligned (may be NULL when 0)
 * Replaces: matmul_tp_persistent + matmul_kernel_tp_persistent,
 *           src/tbik/tree_based_matmul.py:190-277 and :50-187.
 */
int tbik_gemm_bf16(const void* A, int64_t lda,
                   const void* B, int64_t ldb_k, int64_t ldb_n,
                   void* C, int64_t ldc,
                   int M, int N, int K, int leaf_k,
                   const void* bias_or_null,
                   void* workspace, size_t workspace_bytes,
                   tbik_stream_t stream);

/*
 * Bytes of device workspace tbik_gemm_bf16 needs for this problem (0 for small problems).  The
 * large-M kernel parks the upper levels of the merge tree there; its contents are scratch, but two
 * launches that run concurrently must not share it.
 * Replaces: the in-register tensor `S` of the reference kernel, src/tbik/tree_based_matmul.py:85.
 */
size_t tbik_gemm_workspace_bytes(int M, int N, int K, int leaf_k);
/* The same for a row-major B[K,N] (ldb_n == 1); f16 != 0: for tbik_gemm_f16. */
size_t tbik_gemm_workspace_bytes_rowmajor_b(int M, int N, int K, int leaf_k, int f16);
/*
 * How tbik_gemm_bf16 (f16 != 0: tbik_gemm_f16) would run this problem: the decision the workspace size above comes
 * from, for callers and tests that want to see it (host only, launches nothing, no effect on any result).
 *   out5[0] path: 0 one launch with K cut over the waves of a work-group (a few rows), 1 128x128 tiles,
 *                 2 two column regions with a K split each, 3 one grid with one K split
 *   out5[1] K split (of the first region for path 2, 0 if that region runs on 128x128 tiles; waves per strip for path 0)
 *   out5[2] columns of the first region (path 2), else 0
 *   out5[3] K split of the second region (path 2), else 0
 *   out5[4] 1 when both regions go out as one launch
 * Every choice yields the same bits (shard tree o leaf tree = full tree).
 * Replaces: the fixed launch configuration of the reference, src/tbik/tree_based_matmul.py:206-238 (no counterpart
 * for the K split: the reference cuts K only across GPUs).
 */
int tbik_gemm_plan_info(int M, int N, int K, int leaf_k, int f16, int rowmajor_b, int* out5);

/*
 * tbik_gemm_bf16 for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Same arguments (without the workspace), same kernels, same bits; the workspace is
 * a fixed array of TBIK_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process ends.  A
 * problem whose tbik_gemm_workspace_bytes() exceeds that size returns TBIK_ERR_SCRATCH_LIMIT before anything is
 * launched (decode- and mid-sized batches fit, and so does the 2048-row benchmark shape, whose two parked tree levels
 * are 32 MiB; the 4096-row shapes of the 32B configuration do not).  The call allocates and frees
 * nothing.  The first call on a device resolves the array's device address (hipGetSymbolAddress): make that call
 * outside a graph capture.  Every call on a GPU uses that GPU's one array, whose contents are scratch (written
 * before they are read, nothing has to start at zero): two calls that overlap in time on one GPU -- different
 * streams, or two graphs replayed concurrently -- race on it and must be ordered by the caller.
 * No counterpart in the reference (its Triton kernel keeps the merge stack in registers and allocates only its
 * output through torch, src/tbik/tree_based_matmul.py:251).
 */
#define TBIK_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)
int tbik_gemm_bf16_static(const void* A, int64_t lda,
                          const void* B, int64_t ldb_k, int64_t ldb_n,
                          void* C, int64_t ldc,
                          int M, int N, int K, int leaf_k,
                          const void* bias_or_null,
                          tbik_stream_t stream);

/*
 * out[i] = adjacent-pair binary tree over parts[0..nparts-1][i], bf16 adds (round to nearest even
 * at every node); nparts a power of two up to 32; all buffers contiguous, numel elements, 2-byte aligned
 * (16-byte aligned buffers take the vector path).  `out` may alias parts[0].
 * Replaces: the local adds of tree_all_reduce_sum_native, src/tbik/tree_based_all_reduce.py:32-37,
 *           simple_matmul.py:35-38, and packed_tree_reduce / custom_tree_all_reduce,
 *           mini_allreduce/tbik_kernel/csrc/allreduce/custom_all_reduce.cuh:203-234, 301-312.
 */
int tbik_tree_combine_bf16(const void* const* parts, int nparts,
                           void* out, int64_t numel,
                           tbik_stream_t stream);

/*
 * C[M,N] (bf16) = A[M,K] x B[K,N] (+ bias[N] in fp32 before the single rounding), one fp32
 * accumulator per element run strictly sequentially over K by the same MFMA chain for every M
 * (batch invariant).  Layout rules as tbik_gemm_bf16; K only needs to be a multiple of 8.
 * Replaces: matmul_persistent + matmul_kernel_persistent, src/bio/batch_invariant_ops.py:127-197
 *           and :42-124 (aten::mm / aten::addmm overrides, :442-447).
 */
int bi_gemm_bf16(const void* A, int64_t lda,
                 const void* B, int64_t ldb_k, int64_t ldb_n,
                 void* C, int64_t ldc,
                 int M, int N, int K,
                 const void* bias_or_null,
                 tbik_stream_t stream);

/*
 * RMSNorm over the last dimension, bf16 in/out, fp32 arithmetic, one wavefront per row in a fixed
 * lane->element order (row i's result does not depend on `rows`):
 *   x32 = x (+ residual);  residual_out = bf16(x32)          (only when residual != NULL)
 *   out = bf16( bf16(x32 * rsqrt(mean(x32^2) + eps)) * weight )   (weight may be NULL)
 * x/out/residual/residual_out have row stride ld* elements; hidden % 8 == 0.
 * Replaces: patch_rms_norm -> vLLM RMSNorm.forward_native -> aten::mean.dim override,
 *           src/patch/patch_batch_invariant.py:9-16, src/bio/batch_invariant_ops.py:459-472.
 */
int bi_rmsnorm_bf16(const void* x, int64_t ldx,
                    const void* residual_or_null, int64_t ldr,
                    const void* weight_or_null,
                    void* out, int64_t ldo,
                    void* residual_out_or_null, int64_t ldro,
                    int64_t rows, int hidden, float eps,
                    tbik_stream_t stream);

/*
 * Bytes of workspace bi_log_softmax / bi_log_softmax_f32 need for a [rows, cols] input.  (A call of at least 192 rows
 * of at most 154,624 elements whose rows allow 16-byte accesses runs as one launch with the row resident on chip and
 * does not touch the workspace; it may then be NULL.)
 */
size_t bi_log_softmax_workspace_bytes(int64_t rows, int64_t cols);

/*
 * out[r, :] = x[r, :] - max - log(sum(exp(x[r, :] - max))), last dimension, fp32 arithmetic.
 * dtype codes: 0 = fp32, 1 = bf16, 2 = fp16; the output is fp32 or has the input's type (the reference's kernel loads
 * the input dtype directly and the aten override's half_to_float asks for an fp32 result).
 * Every row is cut into fixed 4096-element segments (a function of `cols` only); segment (max, sum) pairs are merged
 * in segment order, so row r's result does not depend on `rows`.  Small batches run as two launches over
 * (row, segment) work-groups with the pairs in `workspace`; from 192 rows on, one work-group per row keeps the row on
 * chip between its one read and its one write -- the same expression, the same bits.  `write_softmax` != 0 writes
 * exp(log_softmax) instead.  ldx / ldo are row strides in elements.
 * Replaces: log_softmax + _log_softmax_kernel, src/bio/batch_invariant_ops.py:263-301 and
 *           :200-260 (aten::_log_softmax / aten::_softmax overrides, :450-456).
 */
int bi_log_softmax(const void* x, int64_t ldx, int in_dtype_code,
                   void* out, int64_t ldo, int out_dtype_code,
                   int64_t rows, int64_t cols,
                   void* workspace, size_t workspace_bytes,
                   int write_softmax,
                   tbik_stream_t stream);

/* bi_log_softmax with fp32 input and output. */
int bi_log_softmax_f32(const void* x, int64_t ldx,
                       void* out, int64_t ldo,
                       int64_t rows, int64_t cols,
                       void* workspace, size_t workspace_bytes,
                       int write_softmax,
                       tbik_stream_t stream);

/*
 * Mean over the middle dimension of a contiguous (outer, n, inner) view, fp32 accumulation in a
 * fixed order that depends only on n and inner; dtype_code: 0 = fp32, 1 = bf16, 2 = fp16 (input
 * and output share it).
 * Replaces: mean_dim + mean_kernel, src/bio/batch_invariant_ops.py:352-439 and :304-349
 *           (aten::mean.dim override, :459-472).
 */
int bi_mean_dim(const void* x, void* out,
                int64_t outer, int64_t n, int64_t inner,
                int dtype_code,
                tbik_stream_t stream);

/*
 * Causal grouped-query attention with a fixed key order (tiles of 32 keys, ascending, online softmax, one
 * pass, no split over keys), bf16, head_dim 128; prefill, chunked prefill and decode run the same arithmetic
 * per row (whichever kernel takes the call), and a token's output does not depend on the batch it is computed in.
 *   q, out      [tokens, q_heads, 128]
 *   k_cache     [batch, kv_heads, max_len, 128]
 *   vt_cache    [batch, kv_heads, 128, max_len]   (V stored transposed; entries behind ctx_len must be finite)
 *   q_start/q_len/ctx_len  device int32 [batch]: first token row, number of new tokens, cache length
 *                          including the new tokens (query r of sequence b sits at position ctx_len-q_len+r)
 * Replaces: the fixed-tile attention of the train/inference alignment patch,
 *           _kernel_unified_attention_2d, src/patch/patch_training_inference_align.py:171-487 (its KV-order
 *           rule, not vLLM's paged-cache plumbing).
 */
int bi_attention_bf16(const void* q, const void* k_cache, const void* vt_cache, void* out,
                      const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                      int batch, int max_q_len, int q_heads, int kv_heads, int head_dim, int max_len,
                      float scale, tbik_stream_t stream);

/*
 * fp16 counterparts of tbik_gemm_bf16 / tbik_gemm_workspace_bytes / tbik_tree_combine_bf16 / bi_gemm_bf16: same
 * arguments and contract, elements are IEEE half, leaves are chains of v_mfma_f32_16x16x32_f16 rounded once to
 * fp16, every tree node is one fp16 addition (round to nearest even).
 * Replaces: the float16 branch of the reference's dtype-keyed configuration,
 *           src/tbik/tree_based_matmul.py:206-238 and src/bio/batch_invariant_ops.py:138-170.
 */
size_t tbik_gemm_f16_workspace_bytes(int M, int N, int K, int leaf_k);
int tbik_gemm_f16(const void* A, int64_t lda,
                  const void* B, int64_t ldb_k, int64_t ldb_n,
                  void* C, int64_t ldc,
                  int M, int N, int K, int leaf_k,
                  const void* bias_or_null,
                  void* workspace, size_t workspace_bytes,
                  tbik_stream_t stream);
int tbik_tree_combine_f16(const void* const* parts, int nparts, void* out, int64_t numel, tbik_stream_t stream);
/*
 * The same adjacent-pair tree over fp32 partials (a node is one fp32 addition; 4-byte aligned buffers, 16-byte
 * aligned ones take the vector path).
 * Replaces: the float instantiation of the reference's tree reduce,
 *           mini_allreduce/tbik_kernel/csrc/allreduce/custom_all_reduce.cuh:203-234 (instantiated for float in custom_all_reduce.cu:118-122), and the
 *           local adds of tree_all_reduce_sum_native on float32 tensors, src/tbik/tree_based_all_reduce.py:32-37.
 */
int tbik_tree_combine_f32(const void* const* parts, int nparts, void* out, int64_t numel, tbik_stream_t stream);
int bi_gemm_f16(const void* A, int64_t lda,
                const void* B, int64_t ldb_k, int64_t ldb_n,
                void* C, int64_t ldc,
                int M, int N, int K,
                const void* bias_or_null,
                tbik_stream_t stream);

/*
 * fp16 counterparts of bi_rmsnorm_bf16 and bi_silu_mul_bf16: same arguments, IEEE half elements, the same places
 * where a value is rounded to the element type.
 */
int bi_rmsnorm_f16(const void* x, int64_t ldx,
                   const void* residual_or_null, int64_t ldr,
                   const void* weight_or_null,
                   void* out, int64_t ldo,
                   void* residual_out_or_null, int64_t ldro,
                   int64_t rows, int hidden, float eps,
                   tbik_stream_t stream);
int bi_silu_mul_f16(const void* gate_up, int64_t ld_in,
                    void* out, int64_t ld_out,
                    int64_t rows, int inter,
                    tbik_stream_t stream);

/*
 * fp32 variants: C[M,N] = A[M,K] x B[K,N] (+ bias), all float.  tbik_gemm_f32 is tree-ordered with leaves of 128
 * (leaf_k must be 128, K a multiple of it): a leaf is the fp32 sum of its products, every tree node one fp32
 * addition; no workspace.  bi_gemm_f32 runs one fp32 accumulator over K (K a multiple of 16; callers pad with
 * zeros).  Products are full-precision fp32 MFMAs in an order that depends on K only.  16-byte aligned A and B,
 * leading dimensions multiples of 4, ldb_k == 1.
 * Replaces: the float32 branch of the reference's dtype-keyed configurations,
 *           src/tbik/tree_based_matmul.py:223-231 and src/bio/batch_invariant_ops.py:160-170.
 */
int tbik_gemm_f32(const void* A, int64_t lda,
                  const void* B, int64_t ldb_k, int64_t ldb_n,
                  void* C, int64_t ldc,
                  int M, int N, int K, int leaf_k,
                  const void* bias_or_null,
                  tbik_stream_t stream);
int bi_gemm_f32(const void* A, int64_t lda,
                const void* B, int64_t ldb_k, int64_t ldb_n,
                void* C, int64_t ldc,
                int M, int N, int K,
                const void* bias_or_null,
                tbik_stream_t stream);

/*
 * Gated activation in front of the row-split down projection:
 *   out[r, i] = bf16( bf16(silu(gate_up[r, i])) * gate_up[r, inter + i] ),  i < inter,  silu in fp32.
 * gate_up [rows, >= 2*inter] with row stride ld_in, out [rows, inter] with row stride ld_out (elements);
 * inter, ld_in, ld_out multiples of 8, 16-byte aligned pointers.  Elementwise (batch invariant).
 * Replaces: the unfused SiluAndMul that produces the input of the patched RowParallelLinear forward
 *           (down_proj), src/patch/patch_tp_invariant.py:10-48; model wiring simple_rl.py:320-338.
 */
int bi_silu_mul_bf16(const void* gate_up, int64_t ld_in,
                     void* out, int64_t ld_out,
                     int64_t rows, int inter,
                     tbik_stream_t stream);

/*
 * Caller side of bi_attention_bf16 for a Qwen3-style block: per-head RMSNorm of q and k (weights [128]), rotary
 * embedding (rotate-half, angle = position * inv_freq[i], fp32), and the KV-cache write, for the fused projection
 * output qkv [tokens, (q_heads + 2*kv_heads) * 128] (row stride ld):
 *   q_out    [tokens, q_heads, 128]
 *   k_cache  [batch, kv_heads, max_len, 128]   row (seq_of_token[t], h, positions[t]) is written
 *   vt_cache [batch, kv_heads, 128, max_len]   column positions[t] is written
 * positions / seq_of_token: device int64 [tokens].  One wavefront per (token, head): batch invariant.
 * Replaces: the rotary-embedding patch of the alignment mode and the engine code around it,
 *           src/patch/patch_training_inference_align.py:35-44; model wiring simple_rl.py:320-338 (qk_norm, head_dim 128).
 */
int bi_qk_norm_rope_cache_bf16(const void* qkv, int64_t ld,
                               const void* q_weight, const void* k_weight,
                               const float* inv_freq,
                               const int64_t* positions, const int64_t* seq_of_token,
                               void* q_out, void* k_cache, void* vt_cache,
                               int64_t tokens, int q_heads, int kv_heads, int head_dim, int max_len, int batch,
                               float eps, tbik_stream_t stream);

/*
 * One decode step of an attention block in one launch: bi_qk_norm_rope_cache_bf16 followed by bi_attention_bf16 for
 * sequences that each bring ONE new token.  Row b of qkv [batch, (q_heads + 2*kv_heads) * 128] (row stride ld) is
 * sequence b's token at position ctx_len[b] - 1 (ctx_len: cache length including it, device int32 [batch]; a sequence
 * with ctx_len <= 0 is skipped).  The work-group of a (sequence, KV head) forms its query heads, the key and the value
 * itself, files key and value in the caches and attends: out [batch, q_heads, 128].  Bit-identical to the two calls
 * (the same per-head function, the same attention kernel).
 * Returns TBIK_ERR_UNSUPPORTED (3), with nothing launched, where the decode attention kernel does not apply (max_len
 * not a multiple of 32, query heads per KV head not 1, 2, 4 or 8): the caller then makes the two calls.
 * Replaces: the rotary-embedding patch and the attention kernel of the alignment mode for a decode step,
 *           src/patch/patch_training_inference_align.py:35-44 and :171-487.
 */
int bi_attention_decode_qkv_bf16(const void* qkv, int64_t ld,
                                 const void* q_weight, const void* k_weight, const float* inv_freq,
                                 void* k_cache, void* vt_cache, void* out,
                                 const int32_t* ctx_len,
                                 int batch, int q_heads, int kv_heads, int head_dim, int max_len,
                                 float scale, float eps, tbik_stream_t stream);

/*
 * Greedy sampling: out[r] (int64) = index of the largest element of row r of x [rows, cols] (bf16, row stride ld
 * elements), ties resolved to the lowest index; the pair order (value, then lowest index) is total, so the result
 * does not depend on how a row is split over lanes.  A NaN is never selected (a row of NaNs gives 0).
 * Replaces: the token choice of the engine that the reference drives (vllm_generate, simple_inference.py:62-105,
 *           which samples inside vLLM and compares per-step log-probabilities); for the greedy decoding of the
 *           end-to-end invariance check the tie rule has to be fixed, which an unordered arg-max does not do.
 */
int bi_argmax_bf16(const void* x, int64_t ld, void* out, int64_t rows, int cols, tbik_stream_t stream);

/*
 * bi_argmax_bf16 plus the bookkeeping of a decode step, in the same launch (a step of a small batch is a chain of
 * short kernels, and each of the four updates below would be one more).  Row r's index goes to next_token[r] (int64)
 * and, where given, to history[r * history_ld + count[r]] (int64; skipped once count[r] reaches history_ld); then
 * count[r] (int64), positions[r] (int64) and ctx_len[r] (int32) advance by one.  history, count, positions and ctx_len
 * may each be NULL (history needs count); all are device arrays of `rows` entries (history: rows x history_ld).
 * Replaces: the sampler output and the per-sequence state update of the engine that the reference drives
 *           (vllm_generate, simple_inference.py:62-105); same token choice as bi_argmax_bf16.
 */
int bi_argmax_advance_bf16(const void* x, int64_t ld, void* next_token, int64_t rows, int cols,
                           void* history, int64_t history_ld, void* count, void* positions, void* ctx_len,
                           tbik_stream_t stream);

/*
 * One-launch compositions for decode-sized batches (a handful of rows): the producer of a matmul's activations runs
 * inside the matmul while it stages them, which saves a launch and a round trip of the activations through memory.
 * Both evaluate exactly the expressions of the two-launch forms (the same device functions, the same MFMA chains and
 * tree), so the results are bit-identical to those and a caller may take either form per call.  Both return
 * TBIK_ERR_UNSUPPORTED (3) when the one-launch kernel does not apply to the shape -- more rows than the work-group can
 * stage, a row-major B, a strip grid that would not balance the chip: the caller then runs the two launches.
 *
 * bi_rmsnorm_gemm_bf16:  C[M,N] = bi_gemm_bf16( bi_rmsnorm_bf16(x [+ residual], norm_weight, eps), B )   (+ bias)
 *   x [M,K] (row stride ldx), residual [M,K] or NULL, norm_weight [K] or NULL; when residual is given, residual_out
 *   [M,K] receives bf16(x + residual) and must not be x or residual themselves (every work-group reads both while
 *   the first one writes it); B = [N,K] K-contiguous (ldb_k == 1).  Applies for K <= 8192 with M * K <= 32768 and
 *   M * (2K + 16) <= 40 KiB (M <= 4 at a hidden size of 4096).
 *   Replaces: RMSNorm.forward_native routed through the batch-invariant mean (src/patch/patch_batch_invariant.py:9-16)
 *             followed by the column-parallel projection through aten::mm (src/bio/batch_invariant_ops.py:442-447).
 *
 * tbik_gemm_silu_mul_bf16:  C[M,N] = tbik_gemm_bf16( act, B, leaf_k )   (+ bias),  act = silu(gate) * up as bi_silu_mul_bf16
 *   gate, up [M,K] with the same row stride ld (the two halves of the merged gate/up projection: up = gate + inter;
 *   a rank's K shard of both halves in a tensor-parallel run), K = the reduction extent of the row-split projection;
 *   B = [N,K] K-contiguous.  Applies where the one-launch few-rows tree kernel does and forming the activations in
 *   every work-group is cheaper than a launch of its own: M <= 4, M * K <= 16384, N <= 4096 (one work-group per CU).
 *   Replaces: SiluAndMul followed by the patched RowParallelLinear forward of down_proj,
 *             src/patch/patch_tp_invariant.py:10-48 (the local matmul of :31).
 */
int bi_rmsnorm_gemm_bf16(const void* x, int64_t ldx,
                         const void* residual_or_null, int64_t ldr,
                         const void* norm_weight_or_null, float eps,
                         void* residual_out_or_null, int64_t ldro,
                         const void* B, int64_t ldb_k, int64_t ldb_n,
                         void* C, int64_t ldc,
                         int M, int N, int K,
                         const void* bias_or_null,
                         tbik_stream_t stream);
int tbik_gemm_silu_mul_bf16(const void* gate, const void* up, int64_t ld,
                            const void* B, int64_t ldb_k, int64_t ldb_n,
                            void* C, int64_t ldc,
                            int M, int N, int K, int leaf_k,
                            const void* bias_or_null,
                            tbik_stream_t stream);

/*
 * The consumer side of a row-split layer in the same launch as the layer's last pass: the (add-)RMSNorm that follows
 * o_proj and down_proj in a decoder block, computed by the kernel that combines the K shards, so the layer's output
 * never goes through memory un-normalised.  Both evaluate exactly the expressions of the separate calls (the shard
 * tree of tbik_tree_combine_bf16 with the bias behind it, then the row function of bi_rmsnorm_bf16), so the results
 * are bit-identical to those.
 *
 * tbik_gemm_rmsnorm_bf16:  out[M,N] = bi_rmsnorm_bf16( tbik_gemm_bf16(A, B, leaf_k) (+ bias) [+ residual], norm_weight, eps )
 *   residual [M,N] or NULL; with a residual, residual_out [M,N] receives bf16(result + residual) (it may be the
 *   residual itself).  workspace as for tbik_gemm_bf16 (tbik_gemm_workspace_bytes of the same M, N, K, leaf_k).
 *   Returns TBIK_ERR_UNSUPPORTED (3), with nothing launched, where the matmul of this shape does not end in one shard
 *   combine over whole rows (a handful of rows: the one-launch kernel; large M: column regions or no K split) or
 *   N > 8192: the caller then runs tbik_gemm_bf16 and bi_rmsnorm_bf16.
 *   Replaces: the patched RowParallelLinear forward (src/patch/patch_tp_invariant.py:10-48) followed by the model's
 *             fused add-RMSNorm routed through the batch-invariant mean (src/patch/patch_batch_invariant.py:9-16).
 *
 * tbik_tree_combine_rmsnorm_bf16:  the same for partials that the caller holds (the ranks' results of a row-split layer
 *   brought to one GPU): parts = nparts (2..32, a power of two) device pointers to contiguous [rows, hidden] arrays,
 *   hidden a multiple of 8 and <= 8192, everything 16-byte aligned.
 *   Replaces: tree_all_reduce_sum (src/tbik/tree_based_all_reduce.py:9-37) followed by that add-RMSNorm.
 */
int tbik_gemm_rmsnorm_bf16(const void* A, int64_t lda,
                           const void* B, int64_t ldb_k, int64_t ldb_n,
                           int M, int N, int K, int leaf_k,
                           const void* bias_or_null,
                           const void* residual_or_null, int64_t ldr,
                           const void* norm_weight_or_null, float eps,
                           void* residual_out_or_null, int64_t ldro,
                           void* out, int64_t ldo,
                           void* workspace, size_t workspace_bytes,
                           tbik_stream_t stream);
int tbik_tree_combine_rmsnorm_bf16(const void* const* parts, int nparts,
                                   int64_t rows, int hidden,
                                   const void* bias_or_null,
                                   const void* residual_or_null, int64_t ldr,
                                   const void* norm_weight_or_null, float eps,
                                   void* residual_out_or_null, int64_t ldro,
                                   void* out, int64_t ldo,
                                   tbik_stream_t stream);

/*
 * bi_gemm_silu_mul_bf16:  out[M, inter] = bi_silu_mul_bf16( bi_gemm_bf16(x, W) )  for the merged gate/up projection
 *   W = [2*inter, K] K-contiguous (row stride ldw; rows 0 .. inter-1 gate, inter .. 2*inter-1 up), x [M,K] (row stride ldx):
 *   the wave that owns 16 columns of `gate` also owns the same 16 columns of `up`, runs the fixed-order pass over K once per
 *   matrix and stores silu(gate) * up -- the consumer inside the producer again.  Both products are rounded to bf16 before
 *   the activation, so the result is bit-identical to the two calls.  inter a multiple of 16, K a multiple of 32, no bias.
 *   Returns TBIK_ERR_UNSUPPORTED (3), with nothing launched, outside 5 .. 64 rows (fewer rows: the tree matmul of down_proj
 *   forms the activation itself, tbik_gemm_silu_mul_bf16; more: the tile kernels, which have no such epilogue): the caller
 *   then makes the two calls.
 *   Replaces: the merged column-parallel projection through aten::mm (src/bio/batch_invariant_ops.py:442-447) followed by
 *             SiluAndMul, in front of the patched down_proj (src/patch/patch_tp_invariant.py:10-48).
 */
int bi_gemm_silu_mul_bf16(const void* x, int64_t ldx,
                          const void* W, int64_t ldw,
                          void* out, int64_t ldo,
                          int M, int inter, int K,
                          tbik_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TBIK_HIP_H */
