// C[M, N] = A[M, K] * W[N, K]^T with fp32 multiply and fp32 accumulate.
// This is the matrix product of the true 32-bit path and the fallback for operand types the
// bf16 MFMA kernels do not take (for instance a weight that the checkpoint stores in fp32 while
// activations are bf16).  No reduced-precision matrix instruction is used: operands stored in
// bf16 are widened (exactly) before they are multiplied.
//
// Many rows (a portion of a prompt), rows of K that start on 16 bytes: tiles of 128 x 128
// outputs on the matrix cores with v_mfma_f32_32x32x2_f32, which multiplies and adds in fp32
// (gemm_mfma32_kernel below).  Many rows otherwise, and kept for comparison: tiles of 64 x 64
// outputs on the vector ALUs, every output summed
// over k = 0..K-1 in that order by one thread.  Few rows (decode steps), where the product is
// bound by reading W once: a wave owns one to four columns of W for all rows, its lanes walk K side by
// side with 16-byte loads (a wave reads 1 KB of a row of W at a time, several such loads in
// flight), every lane keeps a partial sum per output and the 64 partial sums are added in a fixed
// tree at the end.  Within either kernel a row's result does not depend on the number of rows, on
// the row's place in the batch or on the grid; between the kernels the order of the sums differs,
// so results agree to rounding.
//
// Output modes: 0 = store as TO;  1 = add into a fp32 matrix (the residual stream).
#include "common.h"

namespace {
constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

template <typename TA, typename TW, typename TO, int MODE>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const TA* __restrict__ A,
                                                        const TW* __restrict__ W,
                                                        TO* __restrict__ C, int M, int N, int K,
                                                        int lda, int ldc) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tr = tid / 16, tc = tid % 16;  // micro-tile rows tr*4.., cols tc*4..
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  const int lrow = tid / 4, lk = (tid % 4) * 4;  // this thread stages 4 consecutive k of one row
  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      const int m = m0 + lrow;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = k0 + lk + e;
        As[lk + e][lrow] = (m < M && k < K) ? Elem<TA>::load(A + static_cast<size_t>(m) * lda + k)
                                            : 0.f;
      }
      const int n = n0 + lrow;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = k0 + lk + e;
        Ws[lk + e][lrow] = (n < N && k < K) ? Elem<TW>::load(W + static_cast<size_t>(n) * K + k)
                                            : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[TM], w[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[kk][tr * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) w[j] = Ws[kk][tc * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + tr * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tc * TN + j;
      if (n >= N) continue;
      TO* c = C + static_cast<size_t>(m) * ldc + n;
      if (MODE == 1) {
        Elem<TO>::store(c, Elem<TO>::load(c) + acc[i][j]);
      } else {
        Elem<TO>::store(c, acc[i][j]);
      }
    }
  }
}

// Few rows of A (decode steps): a tile of 64 x 64 outputs would leave N / 64 workgroups to stream
// all of W.  Here a workgroup owns 16 columns and 16 rows, one output per thread, and walks K in
// steps of 64 through LDS; every output is still accumulated over k = 0..K-1 in that order by
// one thread with the same fused multiply-adds, so it has the same bits as from the kernel above.
constexpr int RN = 16, RM = 16, RK = 64;

template <typename TA, typename TW, typename TO, int MODE>
__global__ __launch_bounds__(256) void gemm_rows_kernel(const TA* __restrict__ A,
                                                        const TW* __restrict__ W,
                                                        TO* __restrict__ C, int M, int N, int K,
                                                        int lda, int ldc) {
  __shared__ __align__(16) float As[RM][RK + 4];  // rows 16 bytes apart in banks: no conflicts
  __shared__ __align__(16) float Ws[RN][RK + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * RM, n0 = blockIdx.x * RN;
  const int r = tid / RN, c = tid % RN;          // this thread's output
  const int lrow = tid / 16, lk = (tid % 16) * 4;  // and what it stages: 4 consecutive k of a row
  // whole 16-byte loads where both operands are fp32 and every row starts on 16 bytes
  const bool vec = sizeof(TA) == 4 && sizeof(TW) == 4 && K % 4 == 0 && lda % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0;
  float acc = 0.f;
  for (int k0 = 0; k0 < K; k0 += RK) {
    {
      const int m = m0 + lrow, n = n0 + lrow, k = k0 + lk;
      if (vec) {
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f), w = a;
        if (m < M && k < K) a = *reinterpret_cast<const float4*>(A + static_cast<size_t>(m) * lda + k);
        if (n < N && k < K) w = *reinterpret_cast<const float4*>(W + static_cast<size_t>(n) * K + k);
        *reinterpret_cast<float4*>(&As[lrow][lk]) = a;
        *reinterpret_cast<float4*>(&Ws[lrow][lk]) = w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          As[lrow][lk + e] = (m < M && k + e < K) ? Elem<TA>::load(A + static_cast<size_t>(m) * lda + k + e) : 0.f;
          Ws[lrow][lk + e] = (n < N && k + e < K) ? Elem<TW>::load(W + static_cast<size_t>(n) * K + k + e) : 0.f;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < RK; kk += 4) {
      const float4 a = *reinterpret_cast<const float4*>(&As[r][kk]);
      const float4 w = *reinterpret_cast<const float4*>(&Ws[c][kk]);
      acc = fmaf(a.x, w.x, acc);
      acc = fmaf(a.y, w.y, acc);
      acc = fmaf(a.z, w.z, acc);
      acc = fmaf(a.w, w.w, acc);
    }
    __syncthreads();
  }
  const int m = m0 + r, n = n0 + c;
  if (m >= M || n >= N) return;
  TO* o = C + static_cast<size_t>(m) * ldc + n;
  if (MODE == 1) {
    Elem<TO>::store(o, Elem<TO>::load(o) + acc);
  } else {
    Elem<TO>::store(o, acc);
  }
}

// ---- few rows, W streamed once: see the head of the file.
constexpr int SKC = 1024;    // elements of K per staged chunk of A
constexpr int SQ = 4 * KVF_WAVE;  // elements of K a wave reads per step (16 bytes a lane)

template <typename T> struct Quad;
template <> struct Quad<float> {
  static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
};
template <> struct Quad<bf16_t> {
  static __device__ __forceinline__ float4 load(const bf16_t* p) {
    const uint2 r = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                       __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u));
  }
};

// ---- many rows on the matrix cores, true fp32.
// A workgroup of four waves owns 128 x XN outputs; a wave owns 64 x (XN / 2) of them as 32 x 32
// tiles of v_mfma_f32_32x32x2_f32 (lane l supplies A[row l % 32][k = l / 32] and
// W[column l % 32][k = l / 32], and holds 16 outputs of column l % 32).  K is walked in tiles of
// 32: the tile after the current one travels from memory to registers while the matrix cores work
// on the current one from LDS.  Within a tile of 32 the two halves of the wave take k = 8u + e
// and k = 8u + 4 + e in instruction (u, e), so that a lane reads its operands from LDS 16 bytes
// at a time; the order of the sums is fixed by K alone.  Rows of A and W start on 16 bytes
// (8 for bf16) and K is a multiple of 4: the caller checks.
constexpr int XM = 128, XK = 32, XLD = XK + 4;   // LDS rows 144 bytes apart
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <typename TA, typename TW, typename TO, int MODE, int XN>
__global__ __launch_bounds__(256) void gemm_mfma32_kernel(const TA* __restrict__ A,
                                                          const TW* __restrict__ W,
                                                          TO* __restrict__ C, int M, int N, int K,
                                                          int lda, int ldc) {
  constexpr int CT = XN / 64;          // 32-column tiles per wave
  constexpr int WQ = XN / 32;          // float4 of W a thread stages per k-tile
  __shared__ __align__(16) float As[XM][XLD];
  __shared__ __align__(16) float Ws[XN][XLD];
  const int tid = threadIdx.x, lane = tid % KVF_WAVE, wave = tid / KVF_WAVE;
  const int m0 = blockIdx.y * XM, n0 = blockIdx.x * XN;
  const int wm = (wave / 2) * 64, wn = (wave % 2) * (XN / 2);
  const int r32 = lane % 32, half = lane / 32;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);

  f32x16 acc[2][CT];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < CT; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // what this thread stages: row srow + 32 i, elements skq .. skq + 3 of the k-tile
  const int srow = tid / 8, skq = (tid % 8) * 4;
  float4 ra[4], rw[WQ];
  auto fetch = [&](int k0) {
    const int k = k0 + skq;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + srow + 32 * i;
      ra[i] = (m < M && k < K) ? Quad<TA>::load(A + static_cast<size_t>(m) * lda + k) : zero;
    }
#pragma unroll
    for (int i = 0; i < WQ; ++i) {
      const int n = n0 + srow + 32 * i;
      rw[i] = (n < N && k < K) ? Quad<TW>::load(W + static_cast<size_t>(n) * K + k) : zero;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<float4*>(&As[srow + 32 * i][skq]) = ra[i];
#pragma unroll
    for (int i = 0; i < WQ; ++i) *reinterpret_cast<float4*>(&Ws[srow + 32 * i][skq]) = rw[i];
  };

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += XK) {
    __syncthreads();   // the tile before has been read by every wave
    stage();
    __syncthreads();
    if (k0 + XK < K) fetch(k0 + XK);
#pragma unroll
    for (int u = 0; u < XK / 8; ++u) {
      float4 a[2], w[CT];
#pragma unroll
      for (int i = 0; i < 2; ++i) a[i] = *reinterpret_cast<const float4*>(&As[wm + 32 * i + r32][8 * u + 4 * half]);
#pragma unroll
      for (int j = 0; j < CT; ++j) w[j] = *reinterpret_cast<const float4*>(&Ws[wn + 32 * j + r32][8 * u + 4 * half]);
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < CT; ++j) {
            const float av = e == 0 ? a[i].x : e == 1 ? a[i].y : e == 2 ? a[i].z : a[i].w;
            const float wv = e == 0 ? w[j].x : e == 1 ? w[j].y : e == 2 ? w[j].z : w[j].w;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, wv, acc[i][j], 0, 0, 0);
          }
    }
  }
  // output v of a lane: row 8 (v / 4) + 4 (lane / 32) + v % 4 of the tile, column lane % 32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < CT; ++j) {
      const int n = n0 + wn + 32 * j + r32;
      if (n >= N) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm + 32 * i + 8 * (v / 4) + 4 * half + v % 4;
        if (m >= M) continue;
        TO* c = C + static_cast<size_t>(m) * ldc + n;
        if (MODE == 1) {
          Elem<TO>::store(c, Elem<TO>::load(c) + acc[i][j][v]);
        } else {
          Elem<TO>::store(c, acc[i][j][v]);
        }
      }
    }
}

// MT rows per workgroup (1, 2, 4, 8 or 16); SN columns of W per wave, each read DEPTH steps
// ahead, so that SN * DEPTH loads of 16 bytes are in flight per lane: narrow outputs (few
// columns, hence few waves) take one column per wave and look far ahead, wide ones four columns.
// SW waves per workgroup share the staged rows of A: with one column per wave a workgroup of four
// waves would stage all of A for four columns of W and move twice the bytes of W through LDS,
// so narrow outputs get sixteen waves per workgroup.
// The sums do not depend on MT, SN, DEPTH or SW.  Needs K % 4 == 0 and rows of A and W that start on
// 16 bytes (8 for bf16): the caller checks.
template <typename TA, typename TW, typename TO, int MODE, int MT, int SN, int DEPTH, int SW>
__global__ __launch_bounds__(SW * KVF_WAVE) void gemm_stream_kernel(
    const TA* __restrict__ A, const TW* __restrict__ W, TO* __restrict__ C, int M, int N, int K,
    int lda, int ldc) {
  __shared__ __align__(16) float As[MT][SKC];
  const int tid = threadIdx.x, lane = tid % KVF_WAVE, wave = tid / KVF_WAVE;
  const int n0 = (blockIdx.x * SW + wave) * SN, m0 = blockIdx.y * MT;
  float acc[MT][SN];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < SN; ++j) acc[i][j] = 0.f;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  // rows of W this wave reads; columns past N read row N - 1 and are dropped at the end
  const TW* wrow[SN];
#pragma unroll
  for (int j = 0; j < SN; ++j) wrow[j] = W + static_cast<size_t>(min(n0 + j, N - 1)) * K + lane * 4;

  float4 w[DEPTH][SN];   // w[t % DEPTH]: step t of this wave's walk along K
#pragma unroll
  for (int t = 0; t < DEPTH; ++t)
#pragma unroll
    for (int j = 0; j < SN; ++j) w[t][j] = t * SQ + lane * 4 < K ? Quad<TW>::load(wrow[j] + t * SQ) : zero;

  const int steps = (K + SQ - 1) / SQ;
  for (int t0 = 0; t0 < steps; t0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const int t = t0 + u, k = t * SQ;      // uniform
      if (k >= K) break;
      if (k % SKC == 0) {
        __syncthreads();  // the chunk before has been read by every wave
        for (int idx = tid; idx < MT * (SKC / 4); idx += SW * KVF_WAVE) {
          const int row = idx / (SKC / 4), kq = k + (idx % (SKC / 4)) * 4;
          float4 a = zero;
          if (m0 + row < M && kq < K) a = Quad<TA>::load(A + static_cast<size_t>(m0 + row) * lda + kq);
          *reinterpret_cast<float4*>(&As[row][kq - k]) = a;
        }
        __syncthreads();
      }
      float4 cur[SN];
#pragma unroll
      for (int j = 0; j < SN; ++j) cur[j] = w[u][j];
      const int ahead = k + DEPTH * SQ;
#pragma unroll
      for (int j = 0; j < SN; ++j) w[u][j] = ahead + lane * 4 < K ? Quad<TW>::load(wrow[j] + ahead) : zero;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const float4 a = *reinterpret_cast<const float4*>(&As[i][k % SKC + lane * 4]);
#pragma unroll
        for (int j = 0; j < SN; ++j) {
          float v = acc[i][j];
          v = fmaf(a.x, cur[j].x, v);
          v = fmaf(a.y, cur[j].y, v);
          v = fmaf(a.z, cur[j].z, v);
          v = fmaf(a.w, cur[j].w, v);
          acc[i][j] = v;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < SN; ++j) {
      const float total = wave_sum(acc[i][j]);
      const int m = m0 + i, n = n0 + j;
      if (lane == 0 && m < M && n < N) {
        TO* o = C + static_cast<size_t>(m) * ldc + n;
        if (MODE == 1) {
          Elem<TO>::store(o, Elem<TO>::load(o) + total);
        } else {
          Elem<TO>::store(o, total);
        }
      }
    }
}

template <typename TA, typename TW, typename TO, int MODE, int MT>
int launch_stream(const TA* A, const TW* W, TO* C, int M, int N, int K, int lda, int ldc, hipStream_t s) {
#define GO(SN, DEPTH, SW)                                                                        \
  do {                                                                                           \
    dim3 grid((N + SN * SW - 1) / (SN * SW), (M + MT - 1) / MT);                                 \
    hipLaunchKernelGGL((gemm_stream_kernel<TA, TW, TO, MODE, MT, SN, DEPTH, SW>), grid,          \
                       dim3(SW * KVF_WAVE), 0, s, A, W, C, M, N, K, lda, ldc);                   \
  } while (0)
  // about four waves or more per compute unit's SIMD at the widest choice that allows it
  if (N >= 16384) GO(4, 2, 4);
  else if (N >= 6144) GO(2, 4, 8);
  else GO(1, 8, 16);
#undef GO
  return kvf_last_error();
}

constexpr int STREAM_MAX_M = 32;
int g_vector_alus_only = 0;   // tests: many rows through the 64 x 64 tiles of the vector ALUs

// Compute units of the current device, asked once per device.
int compute_units() {
  static int known[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (known[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    known[dev] = n;
  }
  return known[dev];
}

template <typename TA, typename TW, typename TO, int MODE>
int launch(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldc,
           hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  const bool quads = K % 4 == 0 && lda % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(A) % (4 * sizeof(TA)) == 0 &&
                     reinterpret_cast<uintptr_t>(W) % (4 * sizeof(TW)) == 0;
  if (M <= STREAM_MAX_M && quads) {
    const TA* a = static_cast<const TA*>(A);
    const TW* w = static_cast<const TW*>(W);
    TO* c = static_cast<TO*>(C);
    if (M == 1) return launch_stream<TA, TW, TO, MODE, 1>(a, w, c, M, N, K, lda, ldc, s);
    if (M == 2) return launch_stream<TA, TW, TO, MODE, 2>(a, w, c, M, N, K, lda, ldc, s);
    if (M <= 4) return launch_stream<TA, TW, TO, MODE, 4>(a, w, c, M, N, K, lda, ldc, s);
    if (M <= 8) return launch_stream<TA, TW, TO, MODE, 8>(a, w, c, M, N, K, lda, ldc, s);
    return launch_stream<TA, TW, TO, MODE, 16>(a, w, c, M, N, K, lda, ldc, s);
  }
  if (M <= 2 * RM) {
    dim3 rows_grid((N + RN - 1) / RN, (M + RM - 1) / RM);
    hipLaunchKernelGGL((gemm_rows_kernel<TA, TW, TO, MODE>), rows_grid, dim3(256), 0, s,
                       static_cast<const TA*>(A), static_cast<const TW*>(W), static_cast<TO*>(C), M,
                       N, K, lda, ldc);
    return kvf_last_error();
  }
  if (quads && !g_vector_alus_only) {
    // tiles of 128 columns where they still give every compute unit two workgroups, of 64 else
    const int wide = ((N + 127) / 128) * ((M + XM - 1) / XM);
    if (wide >= 2 * compute_units()) {
      dim3 mgrid((N + 127) / 128, (M + XM - 1) / XM);
      hipLaunchKernelGGL((gemm_mfma32_kernel<TA, TW, TO, MODE, 128>), mgrid, dim3(256), 0, s,
                         static_cast<const TA*>(A), static_cast<const TW*>(W), static_cast<TO*>(C),
                         M, N, K, lda, ldc);
    } else {
      dim3 mgrid((N + 63) / 64, (M + XM - 1) / XM);
      hipLaunchKernelGGL((gemm_mfma32_kernel<TA, TW, TO, MODE, 64>), mgrid, dim3(256), 0, s,
                         static_cast<const TA*>(A), static_cast<const TW*>(W), static_cast<TO*>(C),
                         M, N, K, lda, ldc);
    }
    return kvf_last_error();
  }
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  hipLaunchKernelGGL((gemm_tile_kernel<TA, TW, TO, MODE>), grid, dim3(256), 0, s,
                     static_cast<const TA*>(A), static_cast<const TW*>(W), static_cast<TO*>(C), M,
                     N, K, lda, ldc);
  return kvf_last_error();
}
}  // namespace

// For tests that compare the two many-row kernels: nonzero keeps products of many rows on the
// vector ALUs.  Returns the setting before.
KVF_EXPORT int kvf_gemm_generic_vector_alus_only(int on) {
  const int before = g_vector_alus_only;
  g_vector_alus_only = on;
  return before;
}

// a_type / w_type: 0 = fp32, 1 = bf16.  out_mode: 0 = store in a_type... see table below.
//   out_kind 0: store fp32      out_kind 1: store bf16      out_kind 2: add into fp32
KVF_EXPORT int kvf_gemm_generic(const void* A, int a_type, const void* W, int w_type, void* C,
                                int out_kind, int M, int N, int K, int lda, int ldc,
                                hipStream_t s) {
#define CASE(AT, WT, TA, TW)                                                                      \
  if (a_type == AT && w_type == WT) {                                                             \
    if (out_kind == 0) return launch<TA, TW, float, 0>(A, W, C, M, N, K, lda, ldc, s);            \
    if (out_kind == 1) return launch<TA, TW, bf16_t, 0>(A, W, C, M, N, K, lda, ldc, s);           \
    if (out_kind == 2) return launch<TA, TW, float, 1>(A, W, C, M, N, K, lda, ldc, s);            \
  }
  CASE(0, 0, float, float)
  CASE(0, 1, float, bf16_t)
  CASE(1, 0, bf16_t, float)
  CASE(1, 1, bf16_t, bf16_t)
#undef CASE
  return static_cast<int>(hipErrorInvalidValue);
}
