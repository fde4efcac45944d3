// The library's bf16 matrix product (hipBLASLt) for many rows of A, called without a framework
// in between: C[M, N] = A[M, K] * W[N, K]^T with fp32 accumulation, C in bf16 or fp32.
//
// Why this exists: a step that cannot be replayed from a graph (a portion of a prompt, whose
// size changes from step to step) launches every kernel from the host, and four products per
// layer through torch.mm cost 17 us of host time each, more than the device needs for them at a
// few hundred rows.  Here a product's descriptors and its algorithm are made once per shape and
// kept; a call is then a table look-up and one hipblasLtMatmul.
//
// Which algorithm: the first the library's heuristic names, except for row counts that come
// back all the time (the powers of two from 32 to 512: the padded batches of captured decode
// steps).  For those the heuristic's first CANDIDATES answers are timed once, on the operands of
// the shape's first call (into a C of the timing's own if the call adds into its C) and with the
// caches swept before every run, and the fastest is kept: a decode step of 64 sequences at the
// 1B shape goes from 1.72 to 1.54 ms.  A shape whose first call comes under stream capture cannot
// be timed and keeps the heuristic's first answer for good (the engine's captures follow an
// eager step, so its shapes are timed).  Either way a shape's algorithm is settled before its
// first result is handed out, and equal calls give equal bits within a process.
//
// hipBLASLt counts in column-major matrices.  Row-major C[M, N] is column-major C^T[N, M] =
// op(W) * A^T: the first operand is W as a K x N column-major matrix (leading dimension K),
// transposed; the second is A as K x M (leading dimension lda), as it is.
//
// The workspace is allocated once per device by kvf_gemm_library_init, which must be called
// outside stream capture.  A product allocates nothing while its stream is being captured;
// outside capture the first timing of candidates allocates the memory the caches are swept with.
#include "common.h"

#include <hipblaslt/hipblaslt.h>

#include <mutex>
#include <unordered_map>

namespace {
constexpr int MAX_DEVICES = 16;

constexpr int CANDIDATES = 16;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;                  // the one in use
  hipblasLtMatmulAlgo_t others[CANDIDATES];    // what the heuristic named, in its order
  int num_others = 0;
  bool usable = false;
  bool timed = true;                           // false: the candidates are still to be timed
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

// Memory that is overwritten between the timed runs of candidates, so that each run finds the
// weights where a layer's first use finds them: in HBM, not in the 256 MB memory-side cache.
constexpr size_t FLUSH_BYTES = 384u << 20;

struct Device {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  void* flush = nullptr;
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
  // row counts that recur, up to where the heuristic's first answer is as good as any in place
  // (at 2,048 rows the timed choice gained nothing in a whole prefill, at 64 it gains 11% of a
  // decode step): their candidates are worth timing
  const bool recurs = k.M >= 32 && k.M <= 512 && (k.M & (k.M - 1)) == 0;
  hipblasLtMatmulHeuristicResult_t found[CANDIDATES];
  int count = 0;
  const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(dv.handle, p.desc, p.w, p.a, p.c, p.c, pref,
                                                             recurs ? CANDIDATES : 1, found, &count);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS) return p;
  for (int i = 0; i < count && i < CANDIDATES; ++i)
    if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= dv.workspace_bytes)
      p.others[p.num_others++] = found[i].algo;
  if (p.num_others > 0) {
    p.algo = p.others[0];
    p.usable = true;
    p.timed = p.num_others < 2;
  }
  return p;
}

// Runs every candidate on the call's own operands (C is written with the same product each
// time) and keeps the fastest: the best of TIMED_RUNS runs each, every run after the caches have
// been swept, as a model's weights are cold when their layer comes round.  Waits for the stream:
// only outside capture.
constexpr int TIMED_RUNS = 4;

void time_candidates(Device& dv, Plan& p, const void* A, const void* W, void* C, hipStream_t s) {
  p.timed = true;
  if (!dv.flush && hipMalloc(&dv.flush, FLUSH_BYTES) != hipSuccess) {
    dv.flush = nullptr;
    hipGetLastError();
    return;  // no room to sweep the caches with: the heuristic's first answer stays
  }
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    if (e0) hipEventDestroy(e0);
    return;
  }
  const float alpha = 1.f, beta = 0.f;
  float best = 0.f;
  int best_i = -1;
  for (int i = 0; i < p.num_others; ++i) {
    float mine = 0.f;
    bool ok = true;
    for (int r = 0; r <= TIMED_RUNS && ok; ++r) {  // the first run is not counted
      float ms = 0.f;
      ok = hipMemsetAsync(dv.flush, r, FLUSH_BYTES, s) == hipSuccess && hipEventRecord(e0, s) == hipSuccess &&
           hipblasLtMatmul(dv.handle, p.desc, &alpha, W, p.w, A, p.a, &beta, C, p.c, C, p.c, &p.others[i],
                           dv.workspace, dv.workspace_bytes, s) == HIPBLAS_STATUS_SUCCESS &&
           hipEventRecord(e1, s) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
           hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
      if (ok && r > 0 && (r == 1 || ms < mine)) mine = ms;
    }
    if (ok && (best_i < 0 || mine < best)) {
      best = mine;
      best_i = i;
    }
  }
  if (best_i >= 0) p.algo = p.others[best_i];
  hipEventDestroy(e0);
  hipEventDestroy(e1);
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
    if (it->second.usable && !it->second.timed) {
      // The algorithm of a shape is settled before its first result is handed out and never
      // changes afterwards, so equal calls give equal bits within a process.  A call that adds
      // into C is timed on a C of its own; under capture nothing can be timed and the
      // heuristic's first answer stays for good.
      hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
      const bool eager = hipStreamIsCapturing(s, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone;
      void* target = C;
      void* own = nullptr;
      if (eager && accumulate) {
        if (hipMalloc(&own, static_cast<size_t>(M) * ldc * sizeof(float)) != hipSuccess) {
          own = nullptr;
          hipGetLastError();
        }
        target = own;
      }
      if (eager && target) time_candidates(dv, it->second, A, W, target, s);
      it->second.timed = true;
      if (own) hipFree(own);
    }
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
