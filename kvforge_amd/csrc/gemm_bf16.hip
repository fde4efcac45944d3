// C[M, N] = A[M, K] * W[N, K]^T for bf16 operands on the matrix cores (fp32 accumulation),
// built for few rows of A: the weight matrix is streamed once per pass of up to 16*MT rows and
// the kernel is bound by HBM, so all of the chip has to pull on W at once.
//
// One workgroup owns 16 rows of W (16 output columns).  Its waves split K: wave w takes the
// 32-wide k-steps w, w + nw, w + 2nw, ... so neighbouring waves read neighbouring 64-byte pieces
// of the same rows.  Per k-step a lane loads 16 B of W (row lane%16, k-offset 8*(lane/16)) and
// 16 B of each 16-row tile of A (row lane%16, same k-offset) and issues one
// v_mfma_f32_16x16x32_bf16 per tile with W as the first operand, so a lane ends up holding four
// consecutive output columns of one row of C.  Partial sums of the waves are added in wave order
// through LDS.  The number of waves depends on N, K and on how many 16-row tiles a pass holds
// (1, 2, 4 or 8), never on the rows themselves.
//
// out_kind: 0 store fp32, 1 store bf16, 2 add into fp32 (the residual stream).
// K must be a multiple of 8 (16-byte loads); a k-step that passes K loads zeros.
#include "common.h"

namespace {
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 load_frag(const bf16_t* p, bool ok) {
  uint4 r = make_uint4(0u, 0u, 0u, 0u);
  if (ok) r = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, r);
}

// more row tiles per pass mean more registers per lane and more LDS per wave: fewer waves
constexpr int max_waves(int mt) { return mt <= 2 ? 16 : (mt == 4 ? 8 : 4); }

template <int MT, int OUT>
__global__ __launch_bounds__(max_waves(MT) * KVF_WAVE) void gemm_skinny_kernel(const bf16_t* __restrict__ A,
                                                           const bf16_t* __restrict__ W,
                                                           void* __restrict__ Cv, int M, int N,
                                                           int K, int lda, int ldc, int m_base) {
  extern __shared__ float red[];  // [nw][MT][64 lanes][4]
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int nw = blockDim.x / KVF_WAVE;
  const int n0 = blockIdx.x * 16;
  const int r16 = lane % 16, kg = lane / 16;
  int wrow = n0 + r16;
  if (wrow >= N) wrow = N - 1;  // clamped rows are computed and never stored
  const bf16_t* wp = W + static_cast<size_t>(wrow) * K + kg * 8;
  const bf16_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    int arow = m_base + t * 16 + r16;
    if (arow >= M) arow = M - 1;
    ap[t] = A + static_cast<size_t>(arow) * lda + kg * 8;
  }
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int ksteps = (K + 31) / 32;
  int ks = wave;
  // four k-steps in flight per wave
  for (; ks + 3 * nw < ksteps; ks += 4 * nw) {
    bf16x8 wf[4], af[4][MT];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = (ks + u * nw) * 32;
      const bool ok = k + kg * 8 + 8 <= K;
      wf[u] = load_frag(wp + k, ok);
#pragma unroll
      for (int t = 0; t < MT; ++t) af[u][t] = load_frag(ap[t] + k, ok);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], af[u][t], acc[t], 0, 0, 0);
  }
  for (; ks < ksteps; ks += nw) {
    const int k = ks * 32;
    const bool ok = k + kg * 8 + 8 <= K;
    const bf16x8 wf = load_frag(wp + k, ok);
#pragma unroll
    for (int t = 0; t < MT; ++t)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, load_frag(ap[t] + k, ok), acc[t], 0, 0, 0);
  }
  // lane holds C[row m = r16][cols n0 + 4*kg .. +3] of each tile
#pragma unroll
  for (int t = 0; t < MT; ++t)
    *reinterpret_cast<f32x4*>(red + ((wave * MT + t) * KVF_WAVE + lane) * 4) = acc[t];
  __syncthreads();
  for (int item = threadIdx.x; item < MT * KVF_WAVE; item += blockDim.x) {
    const int t = item / KVF_WAVE, l = item % KVF_WAVE;
    f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < nw; ++w)
      s += *reinterpret_cast<const f32x4*>(red + ((w * MT + t) * KVF_WAVE + l) * 4);
    const int m = m_base + t * 16 + l % 16;
    const int n = n0 + 4 * (l / 16);
    if (m >= M) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (n + r >= N) break;
      const size_t idx = static_cast<size_t>(m) * ldc + n + r;
      if (OUT == 0) static_cast<float*>(Cv)[idx] = s[r];
      if (OUT == 1) static_cast<bf16_t*>(Cv)[idx].bits = f32_to_bf16(s[r]);
      if (OUT == 2) static_cast<float*>(Cv)[idx] += s[r];
    }
  }
}

template <int MT>
int launch_mt(const bf16_t* A, const bf16_t* W, void* C, int out_kind, int M, int N, int K,
              int lda, int ldc, int m_base, int nw, hipStream_t s) {
  if (nw > max_waves(MT)) nw = max_waves(MT);
  const dim3 grid((N + 15) / 16), block(nw * KVF_WAVE);
  const size_t lds = static_cast<size_t>(nw) * MT * KVF_WAVE * 4 * sizeof(float);
#define GO(OUT)                                                                                    \
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, OUT>), grid, block, lds, s, A, W, C, M, N, K, lda,   \
                     ldc, m_base)
  if (out_kind == 0) GO(0);
  else if (out_kind == 1) GO(1);
  else GO(2);
#undef GO
  return kvf_last_error();
}
}  // namespace

// Waves per workgroup: enough workgroups x waves to keep every CU streaming, at least one
// k-step per wave, at most 16.
static int pick_waves(int N, int K) {
  const int tiles = (N + 15) / 16, ksteps = (K + 31) / 32;
  int nw = (4096 + tiles - 1) / tiles;
  if (nw > 16) nw = 16;
  if (nw > ksteps) nw = ksteps;
  if (nw < 1) nw = 1;
  return nw;
}

KVF_EXPORT int kvf_gemm_bf16(const void* A, const void* W, void* C, int out_kind, int M, int N,
                             int K, int lda, int ldc, hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8 != 0 || lda % 8 != 0 || out_kind < 0 || out_kind > 2)
    return static_cast<int>(hipErrorInvalidValue);
  const bf16_t* a = static_cast<const bf16_t*>(A);
  const bf16_t* w = static_cast<const bf16_t*>(W);
  const int nw = pick_waves(N, K);
  int err = 0;
  for (int m_base = 0; m_base < M && !err; m_base += 128) {
    const int rows = M - m_base < 128 ? M - m_base : 128;
    if (rows <= 16) err = launch_mt<1>(a, w, C, out_kind, M, N, K, lda, ldc, m_base, nw, s);
    else if (rows <= 32) err = launch_mt<2>(a, w, C, out_kind, M, N, K, lda, ldc, m_base, nw, s);
    else if (rows <= 64) err = launch_mt<4>(a, w, C, out_kind, M, N, K, lda, ldc, m_base, nw, s);
    else err = launch_mt<8>(a, w, C, out_kind, M, N, K, lda, ldc, m_base, nw, s);
  }
  return err;
}
