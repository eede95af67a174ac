/*
 * Plain-C restatement of the tree-ordered matmul and the shard combine.
 *
 * TEST INFRASTRUCTURE ONLY: a checker for the HIP kernels and for the PyTorch restatement in
 * tbik_oracle.py.  It is never linked into, loaded by, or called from the shipped library.
 *
 * It is written independently of tbik_oracle.py (own bf16 rounding on the bit pattern, own
 * binary-counter stack, element at a time) so that agreement between the two is evidence and
 * not a tautology.  Reference lines followed (paths relative to the reference checkout):
 *   leaf value        src/tbik/tree_based_matmul.py:121-136  (fp32 dot over one K chunk, then -> bf16)
 *   tree parameters   src/tbik/tree_based_matmul.py:242-249
 *   merge loop        src/tbik/tree_based_matmul.py:140-174
 *   shard combine     src/tbik/tree_based_all_reduce.py:32-35,
 *                     mini_allreduce/tbik_kernel/csrc/allreduce/custom_all_reduce.cuh:203-234
 *
 * The intra-chunk accumulation order (hardware defined in the reference) is plain left to right
 * here; results are therefore bit-comparable only where every chunk sum is exact in fp32.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round to nearest, ties to even, on the bit pattern; NaN stays NaN (quiet) */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline uint16_t bf16_add(uint16_t a, uint16_t b) {
    return f32_to_bf16(bf16_to_f32(a) + bf16_to_f32(b));
}

/* (T, FLB, LEVEL_K) as src/tbik/tree_based_matmul.py:242-249; returns 0 on success */
int tbik_oracle_tree_params(int K, int leaf, int* T, int* flb, int* level_k) {
    if (leaf <= 0 || K <= 0 || K % leaf) return 1;
    int t = K / leaf, f = t, l = 1;
    while (f > 2 && f % 2 == 0) { f /= 2; l++; }
    *T = t; *flb = f; *level_k = l;
    return 0;
}

/*
 * C[M,N] (bf16, row stride ldc) = tree-ordered A[M,K] * B[K,N].
 * A: element (m,k) at A[m*lda + k];  B: element (k,n) at B[k*ldb_k + n*ldb_n].
 * bias (bf16[N]) may be NULL; it is added in bf16 after the tree (:275-276).
 */
int tbik_oracle_matmul_tree(const uint16_t* A, int64_t lda,
                            const uint16_t* B, int64_t ldb_k, int64_t ldb_n,
                            uint16_t* C, int64_t ldc,
                            int M, int N, int K, int leaf, const uint16_t* bias) {
    int T, flb, level_k;
    if (tbik_oracle_tree_params(K, leaf, &T, &flb, &level_k)) return 1;
    uint16_t* stack = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)level_k);
    int* count = (int*)malloc(sizeof(int) * (size_t)level_k);
    if (!stack || !count) { free(stack); free(count); return 2; }
    for (int m = 0; m < M; m++) {
        for (int n = 0; n < N; n++) {
            memset(count, 0, sizeof(int) * (size_t)level_k);
            uint16_t acc = 0;
            for (int j = 0; j < T; j++) {
                float s = 0.0f;
                for (int k = j * leaf; k < (j + 1) * leaf; k++)
                    s += bf16_to_f32(A[m * lda + k]) * bf16_to_f32(B[k * ldb_k + n * ldb_n]);
                acc = f32_to_bf16(s);
                for (int level = 0; level < level_k; level++) {
                    int added = count[level] + 1;
                    int full = (level == 0 ? flb : 2) == added;
                    if (added > 1) acc = bf16_add(stack[level], acc);
                    count[level] = full ? 0 : added;
                    if (!full) { stack[level] = acc; break; }
                }
            }
            if (bias) acc = bf16_add(acc, bias[n]);
            C[m * ldc + n] = acc;
        }
    }
    free(stack); free(count);
    return 0;
}

/* out[i] = adjacent-pair tree over parts[0..nparts-1][i]; nparts a power of two */
int tbik_oracle_tree_combine(const uint16_t* const* parts, int nparts, uint16_t* out, int64_t numel) {
    if (nparts <= 0 || (nparts & (nparts - 1))) return 1;
    uint16_t* tmp = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)nparts);
    if (!tmp) return 2;
    for (int64_t i = 0; i < numel; i++) {
        for (int p = 0; p < nparts; p++) tmp[p] = parts[p][i];
        for (int step = 1; step < nparts; step <<= 1)
            for (int left = 0; left < nparts; left += 2 * step)
                tmp[left] = bf16_add(tmp[left], tmp[left + step]);
        out[i] = tmp[0];
    }
    free(tmp);
    return 0;
}
