/*
 * A host written in plain C against include/tbik_hip.h and the HIP runtime only (no Python, no torch): what a
 * maintainer of a C or cgo/JNI-style binding would write.  It checks, through the C ABI alone,
 *   1. the tree matmul of [M,K] x [K,N] against a double-precision product (within 2^-6 of the output scale),
 *   2. that four K shards combined by tbik_tree_combine_bf16 give the bits of the unsharded call (the property
 *      simple_matmul.py:23-43 of the reference tests with `== 0.0`),
 *   3. that a row computed alone has the bits it has inside the batch (simple_matmul.py:16-20),
 *   4. that the entry point without a workspace (tbik_gemm_bf16_static, for callers that cannot allocate) gives the
 *      bits of the one with a workspace.
 * Exit status 0 when all four hold.  Built by tests/c_host/Makefile with gcc; run by the GPU test suite.
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tbik_hip.h"

#define CHECK_HIP(x)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (x);                                                               \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)

#define CHECK_TBIK(x)                                                                \
  do {                                                                               \
    int rc_ = (x);                                                                   \
    if (rc_ != TBIK_OK) {                                                            \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, tbik_error_string(rc_)); \
      return 2;                                                                      \
    }                                                                                \
  } while (0)

static uint16_t bf16_from_float(float f) { /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static float bf16_to_float(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint32_t lcg_state = 12345u;
static float uniform_pm1(void) { /* deterministic, in (-1, 1) */
  lcg_state = lcg_state * 1664525u + 1013904223u;
  return ((float)(lcg_state >> 8) / 8388608.0f) - 1.0f;
}

int main(void) {
  enum { M = 64, N = 512, K = 4096, LEAF = 256, TP = 4, ROW = 5 };
  const size_t a_bytes = (size_t)M * K * 2, b_bytes = (size_t)N * K * 2, c_bytes = (size_t)M * N * 2;
  uint16_t* A = (uint16_t*)malloc(a_bytes);
  uint16_t* B = (uint16_t*)malloc(b_bytes); /* [N,K], K contiguous: the nn.Linear weight layout */
  uint16_t* C = (uint16_t*)malloc(c_bytes);
  uint16_t* C_tp = (uint16_t*)malloc(c_bytes);
  uint16_t* C_row = (uint16_t*)malloc((size_t)N * 2);
  uint16_t* C_static = (uint16_t*)malloc(c_bytes);
  if (!A || !B || !C || !C_tp || !C_row || !C_static) return 2;
  for (size_t i = 0; i < (size_t)M * K; i++) A[i] = bf16_from_float(uniform_pm1());
  for (size_t i = 0; i < (size_t)N * K; i++) B[i] = bf16_from_float(0.05f * uniform_pm1());

  printf("tbik C ABI version %d\n", tbik_abi_version());
  int T = 0, flb = 0, level_k = 0;
  CHECK_TBIK(tbik_tree_params(K, LEAF, &T, &flb, &level_k));
  printf("K=%d leaf=%d: %d leaves, groups of %d, %d levels\n", K, LEAF, T, flb, level_k);

  void *dA, *dB, *dC, *dRow, *dParts[TP], *dWs = NULL;
  CHECK_HIP(hipMalloc(&dA, a_bytes));
  CHECK_HIP(hipMalloc(&dB, b_bytes));
  CHECK_HIP(hipMalloc(&dC, c_bytes));
  CHECK_HIP(hipMalloc(&dRow, (size_t)N * 2));
  for (int r = 0; r < TP; r++) CHECK_HIP(hipMalloc(&dParts[r], c_bytes));
  CHECK_HIP(hipMemcpy(dA, A, a_bytes, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dB, B, b_bytes, hipMemcpyHostToDevice));
  /* one workspace, large enough for every call below */
  size_t ws = tbik_gemm_workspace_bytes(M, N, K, LEAF);
  const size_t ws_shard = tbik_gemm_workspace_bytes(M, N, K / TP, LEAF), ws_row = tbik_gemm_workspace_bytes(1, N, K, LEAF);
  if (ws_shard > ws) ws = ws_shard;
  if (ws_row > ws) ws = ws_row;
  if (ws) CHECK_HIP(hipMalloc(&dWs, ws));
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));

  /* 1. the whole product */
  CHECK_TBIK(tbik_gemm_bf16(dA, K, dB, 1, K, dC, N, M, N, K, LEAF, NULL, dWs, ws, stream));
  /* 2. four K shards (a rank's slice of the activations and of the row-split weight), then the shard tree */
  for (int r = 0; r < TP; r++) {
    const char* a_r = (const char*)dA + (size_t)r * (K / TP) * 2;
    const char* b_r = (const char*)dB + (size_t)r * (K / TP) * 2;
    CHECK_TBIK(tbik_gemm_bf16(a_r, K, b_r, 1, K, dParts[r], N, M, N, K / TP, LEAF, NULL, dWs, ws, stream));
  }
  CHECK_TBIK(tbik_tree_combine_bf16((const void* const*)dParts, TP, dParts[0], (int64_t)M * N, stream));
  /* 3. one row alone */
  CHECK_TBIK(tbik_gemm_bf16((const char*)dA + (size_t)ROW * K * 2, K, dB, 1, K, dRow, N, 1, N, K, LEAF, NULL, dWs, ws, stream));
  CHECK_HIP(hipStreamSynchronize(stream));
  /* 4. the same product through the entry point that allocates nothing and takes no workspace (into shard buffer 1) */
  CHECK_TBIK(tbik_gemm_bf16_static(dA, K, dB, 1, K, dParts[1], N, M, N, K, LEAF, NULL, stream));
  CHECK_HIP(hipStreamSynchronize(stream));
  CHECK_HIP(hipMemcpy(C_static, dParts[1], c_bytes, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(C, dC, c_bytes, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(C_tp, dParts[0], c_bytes, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(C_row, dRow, (size_t)N * 2, hipMemcpyDeviceToHost));

  int failures = 0;
  /* against the exact product: every node of the tree rounds to bf16 (8 significant bits), so an output is within a
   * few rounding steps of values up to the output scale; 2^-6 of the largest magnitude is a loose bound that a wrong
   * operand, stride or tree still misses by far */
  double scale = 0.0, worst = 0.0;
  double* exact = (double*)malloc((size_t)M * N * sizeof(double));
  if (!exact) return 2;
  for (int m = 0; m < M; m++)
    for (int n = 0; n < N; n++) {
      double s = 0.0;
      for (int k = 0; k < K; k++) s += (double)bf16_to_float(A[(size_t)m * K + k]) * (double)bf16_to_float(B[(size_t)n * K + k]);
      exact[(size_t)m * N + n] = s;
      if (fabs(s) > scale) scale = fabs(s);
    }
  for (size_t i = 0; i < (size_t)M * N; i++) {
    const double d = fabs((double)bf16_to_float(C[i]) - exact[i]);
    if (d > worst) worst = d;
  }
  printf("1. tree matmul against the exact product: max difference %.4g, output scale %.4g\n", worst, scale);
  if (!(worst <= scale / 64.0)) {
    printf("   FAILED: more than 2^-6 of the output scale\n");
    failures++;
  }
  const int tp_equal = memcmp(C, C_tp, c_bytes) == 0;
  printf("2. %d K shards + shard tree %s the unsharded call\n", TP, tp_equal ? "have the bits of" : "DIFFER from");
  failures += !tp_equal;
  const int row_equal = memcmp(C + (size_t)ROW * N, C_row, (size_t)N * 2) == 0;
  printf("3. row %d alone %s the same row inside the batch of %d\n", ROW, row_equal ? "has the bits of" : "DIFFERS from", M);
  failures += !row_equal;
  const int static_equal = memcmp(C, C_static, c_bytes) == 0;
  printf("4. the entry point without a workspace %s the one with a workspace\n", static_equal ? "has the bits of" : "DIFFERS from");
  failures += !static_equal;

  CHECK_HIP(hipStreamDestroy(stream));
  if (dWs) CHECK_HIP(hipFree(dWs));
  for (int r = 0; r < TP; r++) CHECK_HIP(hipFree(dParts[r]));
  CHECK_HIP(hipFree(dRow));
  CHECK_HIP(hipFree(dC));
  CHECK_HIP(hipFree(dB));
  CHECK_HIP(hipFree(dA));
  free(exact);
  free(C_static);
  free(C_row);
  free(C_tp);
  free(C);
  free(B);
  free(A);
  printf(failures ? "FAILED\n" : "ok\n");
  return failures ? 1 : 0;
}
