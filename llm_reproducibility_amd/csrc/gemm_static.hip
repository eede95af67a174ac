// tbik_gemm_bf16_static: the tree-ordered GEMM for callers that cannot allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).  Same kernels and the same bits as tbik_gemm_bf16;
// the workspace (K-shard partials, parked tree levels) is a fixed device array of this library instead of a caller
// buffer.  The array, the per-device table of its addresses and the entry point live in this one file.
#include "common.h"

namespace tbik {
int gemm_dispatch(bool tree, bool f16, const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                  int64_t ldc, int M, int N, int K, int leaf_k, const void* bias, void* ws, size_t ws_bytes,
                  hipStream_t stream);
size_t gemm_workspace_bytes(int M, int N, int K, int leaf_k, bool f16, bool rowmajor_b = false);
}  // namespace tbik

// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.  In host
// code the name is only a handle for hipGetSymbolAddress: the device address it yields is what kernels, copies and
// fills take.
static __device__ __align__(256) unsigned char scratch[TBIK_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];          // device address of `scratch` on device d, valid once bit d of g_ready is set
std::atomic<uint64_t> g_ready{0};

// Address of the current device's copy of `scratch`; resolved once per device, with that device current.
int scratch_for_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return tbik::hip_code(e);
  if (dev < 0 || dev >= kMaxDevices) return TBIK_ERR_UNSUPPORTED;
  const uint64_t bit = 1ull << dev;
  if (!(g_ready.load(std::memory_order_acquire) & bit)) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return tbik::hip_code(e);
    if (!p) return TBIK_ERR_INVALID;
    g_scratch_ptr[dev] = p;  // two threads racing here store the same value
    g_ready.fetch_or(bit, std::memory_order_release);
  }
  *out = g_scratch_ptr[dev];
  return TBIK_OK;
}
}  // namespace

extern "C" int tbik_gemm_bf16_static(const void* A, int64_t lda, const void* B, int64_t ldb_k, int64_t ldb_n, void* C,
                                     int64_t ldc, int M, int N, int K, int leaf_k, const void* bias_or_null,
                                     tbik_stream_t stream) {
  if (M < 0 || N < 0 || K <= 0) return TBIK_ERR_INVALID;
  if (M == 0 || N == 0) return TBIK_OK;
  const size_t need = tbik::gemm_workspace_bytes(M, N, K, leaf_k, false, ldb_k != 1);
  if (need > (size_t)TBIK_STATIC_SCRATCH_BYTES) return TBIK_ERR_SCRATCH_LIMIT;  // before anything is launched
  void* ws = nullptr;
  if (need > 0) {
    const int rc = scratch_for_current_device(&ws);
    if (rc != TBIK_OK) return rc;
  }
  return tbik::gemm_dispatch(true, false, A, lda, B, ldb_k, ldb_n, C, ldc, M, N, K, leaf_k, bias_or_null, ws,
                             need > 0 ? (size_t)TBIK_STATIC_SCRATCH_BYTES : 0, static_cast<hipStream_t>(stream));
}
