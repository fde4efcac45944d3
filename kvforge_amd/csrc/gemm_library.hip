// The library's bf16 matrix product (hipBLASLt) for many rows of A, called without a framework
// in between: C[M, N] = A[M, K] * W[N, K]^T with fp32 accumulation, C in bf16 or fp32.
//
// Why this exists: a step that cannot be replayed from a graph (a portion of a prompt, whose
// size changes from step to step) launches every kernel from the host, and four products per
// layer through torch.mm cost 17 us of host time each, more than the device needs for them at a
// few hundred rows.  Here a product's descriptors and the algorithm the library's heuristic
// picks are made once per shape and kept; a call is then a table look-up and one
// hipblasLtMatmul.
//
// hipBLASLt counts in column-major matrices.  Row-major C[M, N] is column-major C^T[N, M] =
// op(W) * A^T: the first operand is W as a K x N column-major matrix (leading dimension K),
// transposed; the second is A as K x M (leading dimension lda), as it is.
//
// The workspace is allocated once per device by kvf_gemm_library_init, which must be called
// outside stream capture; the product itself allocates nothing and may be captured.
#include "common.h"

#include <hipblaslt/hipblaslt.h>

#include <mutex>
#include <unordered_map>

namespace {
constexpr int MAX_DEVICES = 16;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  bool usable = false;
};

struct Key {
  int M, N, K, lda, ldc, out_f32;
  bool operator==(const Key& o) const {
    return M == o.M && N == o.N && K == o.K && lda == o.lda && ldc == o.ldc && out_f32 == o.out_f32;
  }
};
struct KeyHash {
  size_t operator()(const Key& k) const {
    size_t h = 1469598103934665603ull;
    for (int v : {k.M, k.N, k.K, k.lda, k.ldc, k.out_f32}) h = (h ^ static_cast<size_t>(v)) * 1099511628211ull;
    return h;
  }
};

struct Device {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  std::unordered_map<Key, Plan, KeyHash> plans;
};
Device g_dev[MAX_DEVICES];
std::mutex g_lock;

// Descriptors and algorithm of one shape; `usable` stays false where the library has nothing.
Plan make_plan(Device& dv, const Key& k) {
  Plan p;
  const hipDataType out_t = k.out_f32 ? HIP_R_32F : HIP_R_16BF;
  const hipblasOperation_t t = HIPBLAS_OP_T, n = HIPBLAS_OP_N;
  bool ok = hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &t, sizeof(t)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &n, sizeof(n)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, k.K, k.N, k.K) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, k.K, k.M, k.lda) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&p.c, out_t, k.N, k.M, k.ldc) == HIPBLAS_STATUS_SUCCESS;
  if (!ok) return p;
  hipblasLtMatmulPreference_t pref = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return p;
  const uint64_t room = dv.workspace_bytes;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof(room));
  hipblasLtMatmulHeuristicResult_t found[1];
  int count = 0;
  const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(dv.handle, p.desc, p.w, p.a, p.c, p.c, pref, 1,
                                                             found, &count);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st == HIPBLAS_STATUS_SUCCESS && count > 0 && found[0].state == HIPBLAS_STATUS_SUCCESS &&
      found[0].workspaceSize <= dv.workspace_bytes) {
    p.algo = found[0].algo;
    p.usable = true;
  }
  return p;
}
}  // namespace

// Creates the library handle and the workspace of the current device (once; later calls return
// at once).  Not to be called while a stream is being captured.
KVF_EXPORT int kvf_gemm_library_init(long workspace_bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return static_cast<int>(hipErrorInvalidDevice);
  std::lock_guard<std::mutex> hold(g_lock);
  Device& dv = g_dev[dev];
  if (dv.handle) return 0;
  hipblasLtHandle_t h = nullptr;
  if (hipblasLtCreate(&h) != HIPBLAS_STATUS_SUCCESS) return static_cast<int>(hipErrorNotInitialized);
  void* ws = nullptr;
  if (workspace_bytes > 0 && hipMalloc(&ws, static_cast<size_t>(workspace_bytes)) != hipSuccess) {
    hipblasLtDestroy(h);
    return static_cast<int>(hipErrorOutOfMemory);
  }
  dv.workspace = ws;
  dv.workspace_bytes = ws ? static_cast<size_t>(workspace_bytes) : 0;
  dv.handle = h;
  return 0;
}

// C = A * W^T (accumulate: C += A * W^T; fp32 C only).  A: bf16 [M, K], row stride lda; W: bf16
// [N, K] contiguous; C: [M, N] bf16 or fp32 (out_f32), row stride ldc.  Returns 0, a HIP error
// code, or -1 where the library offers no algorithm for the shape (the caller takes another
// route).  One workspace per device: products on one device must not overlap in time.
KVF_EXPORT int kvf_gemm_library_bf16(const void* A, const void* W, void* C, int out_f32, int accumulate,
                                     int M, int N, int K, int lda, int ldc, hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N || (accumulate && !out_f32) || !A || !W || !C)
    return static_cast<int>(hipErrorInvalidValue);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return static_cast<int>(hipErrorInvalidDevice);
  Plan plan;
  void* ws = nullptr;
  size_t ws_bytes = 0;
  hipblasLtHandle_t handle = nullptr;
  {
    std::lock_guard<std::mutex> hold(g_lock);
    Device& dv = g_dev[dev];
    if (!dv.handle) return static_cast<int>(hipErrorNotInitialized);
    const Key key{M, N, K, lda, ldc, out_f32 ? 1 : 0};
    auto it = dv.plans.find(key);
    if (it == dv.plans.end()) it = dv.plans.emplace(key, make_plan(dv, key)).first;
    plan = it->second;
    ws = dv.workspace;
    ws_bytes = dv.workspace_bytes;
    handle = dv.handle;
  }
  if (!plan.usable) return -1;
  const float alpha = 1.f, beta = accumulate ? 1.f : 0.f;
  const hipblasStatus_t st = hipblasLtMatmul(handle, plan.desc, &alpha, W, plan.w, A, plan.a, &beta, C, plan.c,
                                             C, plan.c, &plan.algo, ws, ws_bytes, s);
  return st == HIPBLAS_STATUS_SUCCESS ? 0 : static_cast<int>(hipErrorLaunchFailure);
}
