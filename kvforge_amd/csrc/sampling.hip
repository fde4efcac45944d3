// Token selection from fp32 logits, one workgroup of 16 waves per row (several for greedy rows).
//
//   temperature == 0      : argmax, the lowest index among equal maxima.
//   temperature  > 0      : z = logits / temperature; optional top-k, then optional top-p on the
//                           renormalised top-k set; p = softmax over what is kept (fp32);
//                           the token is the first index, in vocabulary order, whose cumulative
//                           probability exceeds u * total, u in [0, 1) given by the caller.
// top-k keeps every value >= the k-th largest (equal values are kept together); top-p keeps a
// value iff the mass of strictly larger kept values is below top_p, so the largest is always kept.
// Both thresholds are found by bisection over the order-preserving integer image of a float,
// which needs no sort and no memory beyond the row itself.
#include "common.h"

namespace {
constexpr int THREADS = 1024, NWAVES = THREADS / KVF_WAVE;

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ float block_reduce_sum(float v, float* sh) {
  v = wave_sum(v);
  __syncthreads();
  if (threadIdx.x % KVF_WAVE == 0) sh[threadIdx.x / KVF_WAVE] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NWAVES; ++i) t += sh[i];
  return t;
}
__device__ __forceinline__ float block_reduce_max(float v, float* sh) {
  v = wave_max(v);
  __syncthreads();
  if (threadIdx.x % KVF_WAVE == 0) sh[threadIdx.x / KVF_WAVE] = v;
  __syncthreads();
  float t = -INFINITY;
#pragma unroll
  for (int i = 0; i < NWAVES; ++i) t = fmaxf(t, sh[i]);
  return t;
}

// Greedy rows may be cut into `splits` chunks, one workgroup each (blockIdx.y): a row of a large
// vocabulary is then read by several compute units.  Every workgroup leaves the best of its chunk
// in `work` and takes a ticket; the one that takes the row's last ticket picks the best of the
// chunks in chunk order (so equal maxima still give the lowest index) and puts the tickets back
// to zero.  Nobody waits for anybody.  `work` (int32): [rows] tickets, zero before the first
// launch; [rows * splits] values; [rows * splits] indices.  Rows that sample are done by the
// workgroup of chunk 0 alone.
__global__ __launch_bounds__(THREADS) void sample_kernel(
    const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ u,
    const int* __restrict__ u_step, int u_stride,
    int* __restrict__ tokens, int* __restrict__ work) {
  __shared__ float sh[NWAVES];
  __shared__ float seg_sum[NWAVES];
  __shared__ int sh_idx[NWAVES];
  __shared__ int result;
  const int row = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % KVF_WAVE, wave = tid / KVF_WAVE;
  const float* x = logits + static_cast<size_t>(row) * ld;
  const float temp = temperature[row];

  if (!(temp > 0.f)) {  // greedy
    const int splits = gridDim.y, rows = gridDim.x;
    // chunks of whole groups of four elements
    const int chunk = ((V + splits - 1) / splits + 3) & ~3;
    const int lo = min(V, static_cast<int>(blockIdx.y) * chunk), hi = min(V, lo + chunk);
    float best = -INFINITY;
    int bi = V;
    // rows of 4 floats at a time where the row is 16-byte aligned; several loads in flight
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    const int a4 = lo / 4, b4 = vec ? hi / 4 : a4;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    for (int i0 = a4 + tid; i0 < b4; i0 += 4 * THREADS) {
      float4 r[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        r[u] = i0 + u * THREADS < b4 ? x4[i0 + u * THREADS] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int base = 4 * (i0 + u * THREADS);
        const float e[4] = {r[u].x, r[u].y, r[u].z, r[u].w};
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (e[c] > best || (e[c] == best && base + c < bi)) { best = e[c]; bi = base + c; }
      }
    }
    for (int i = 4 * b4 + tid; i < hi; i += THREADS) {
      const float v = x[i];
      if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    }
    for (int o = KVF_WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, KVF_WAVE);
      const int oi = __shfl_xor(bi, o, KVF_WAVE);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (lane == 0) { sh[wave] = best; sh_idx[wave] = bi; }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < NWAVES; ++w)
        if (sh[w] > best || (sh[w] == best && sh_idx[w] < bi)) { best = sh[w]; bi = sh_idx[w]; }
      if (splits == 1) {
        tokens[row] = bi < V ? bi : 0;
      } else {
        int* vals = work + rows;
        int* idxs = vals + rows * splits;
        const int slot = row * splits + blockIdx.y;
        __hip_atomic_store(vals + slot, __float_as_int(best), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(idxs + slot, bi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __threadfence();  // the chunk's best is visible to the device before the ticket is taken
        const int ticket = atomicAdd(work + row, 1);
        if (ticket == splits - 1) {
          __threadfence();
          best = -INFINITY;
          bi = V;
          for (int c = 0; c < splits; ++c) {
            const float v = __int_as_float(
                __hip_atomic_load(vals + row * splits + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            const int i = __hip_atomic_load(idxs + row * splits + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (v > best || (v == best && i < bi)) { best = v; bi = i; }
          }
          tokens[row] = bi < V ? bi : 0;
          __hip_atomic_store(work + row, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    return;
  }
  if (blockIdx.y != 0) return;

  const float inv_t = 1.f / temp;
  float mx = -INFINITY;
  for (int i = tid; i < V; i += THREADS) mx = fmaxf(mx, x[i] * inv_t);
  mx = block_reduce_max(mx, sh);

  // ---- top-k: key of the k-th largest value (0 keeps everything)
  uint32_t key_min = 0;
  const int k = top_k ? top_k[row] : 0;
  if (k > 0 && k < V) {
    uint32_t t = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = t | (1u << bit);
      float cnt = 0.f;
      for (int i = tid; i < V; i += THREADS) cnt += order_key(x[i] * inv_t) >= cand ? 1.f : 0.f;
      cnt = block_reduce_sum(cnt, sh);
      if (cnt >= static_cast<float>(k)) t = cand;
    }
    key_min = t;
  }
  // ---- top-p on the top-k set
  const float pp = top_p ? top_p[row] : 1.f;
  if (pp < 1.f) {
    float z = 0.f;
    for (int i = tid; i < V; i += THREADS) {
      const float s = x[i] * inv_t;
      if (order_key(s) >= key_min) z += expf(s - mx);
    }
    z = block_reduce_sum(z, sh);
    const float limit = pp * z;
    // largest t with mass(key > t) >= limit; everything with key > t is then kept
    uint32_t t = 0;
    bool any_false = false;
    {
      float f = 0.f;
      for (int i = tid; i < V; i += THREADS) {
        const float s = x[i] * inv_t;
        const uint32_t kk = order_key(s);
        if (kk >= key_min && kk > 0u) f += expf(s - mx);
      }
      f = block_reduce_sum(f, sh);
      any_false = f >= limit;
    }
    if (any_false) {
      for (int bit = 31; bit >= 0; --bit) {
        const uint32_t cand = t | (1u << bit);
        float f = 0.f;
        for (int i = tid; i < V; i += THREADS) {
          const float s = x[i] * inv_t;
          const uint32_t kk = order_key(s);
          if (kk >= key_min && kk > cand) f += expf(s - mx);
        }
        f = block_reduce_sum(f, sh);
        if (f >= limit) t = cand;
      }
      if (t + 1u > key_min) key_min = t + 1u;
    }
  }

  // ---- inverse CDF in vocabulary order: wave w owns a contiguous segment
  const int seg = (V + NWAVES - 1) / NWAVES;
  const int s0 = wave * seg;
  const int s1 = s0 + seg < V ? s0 + seg : V;
  float part = 0.f;
  for (int i = s0 + lane; i < s1; i += KVF_WAVE) {
    const float s = x[i] * inv_t;
    if (order_key(s) >= key_min) part += expf(s - mx);
  }
  part = wave_sum(part);
  if (tid == 0) result = -1;
  if (lane == 0) seg_sum[wave] = part;
  __syncthreads();
  float before = 0.f, total = 0.f;
  for (int w = 0; w < NWAVES; ++w) {
    if (w < wave) before += seg_sum[w];
    total += seg_sum[w];
  }
  const float target = u[(u_step ? *u_step * u_stride : 0) + row] * total;
  // the wave whose segment holds the target walks it; the last wave with mass catches overshoot
  const bool mine = part > 0.f && target >= before && (target < before + part);
  if (mine) {
    float running = before;
    int found = -1, last_kept = -1;
    for (int base = s0; base < s1 && found < 0; base += KVF_WAVE) {
      const int i = base + lane;
      float p = 0.f;
      if (i < s1) {
        const float s = x[i] * inv_t;
        if (order_key(s) >= key_min) p = expf(s - mx);
      }
      float incl = p;
#pragma unroll
      for (int o = 1; o < KVF_WAVE; o <<= 1) {
        const float n = __shfl_up(incl, o, KVF_WAVE);
        if (lane >= o) incl += n;
      }
      const bool hit = p > 0.f && (running + incl > target);
      const unsigned long long hits = __ballot(hit);
      const unsigned long long kept = __ballot(p > 0.f);
      if (hits) found = base + __ffsll(static_cast<long long>(hits)) - 1;
      if (kept) last_kept = base + 63 - __clzll(static_cast<long long>(kept));
      running += __shfl(incl, KVF_WAVE - 1, KVF_WAVE);
    }
    if (found < 0) found = last_kept;
    if (lane == 0) result = found;
  }
  __syncthreads();
  if (tid == 0) {
    int r = result;
    if (r < 0) {
      // rounding left the target past every segment's end: take the last kept token
      for (int i = V - 1; i >= 0; --i)
        if (order_key(x[i] * inv_t) >= key_min) { r = i; break; }
      if (r < 0) r = 0;
    }
    tokens[row] = r;
  }
}
}  // namespace

// u_step (may be null): a device counter; row r then draws with u[*u_step * u_stride + r], so
// that a captured launch can be replayed for several decode steps, each with numbers of its own.
// work (may be null) with splits > 1: greedy rows are read by `splits` workgroups each; it holds
// rows * (1 + 2 * splits) int32, the first `rows` of them zero, and is left so.  Launches that
// share it must not overlap.
KVF_EXPORT int kvf_sample(const float* logits, int ld, int rows, int V, const float* temperature,
                          const int* top_k, const float* top_p, const float* u, const int* u_step,
                          int u_stride, int* tokens, int* work, int splits, hipStream_t s) {
  if (rows <= 0) return 0;
  if (V <= 0 || ld < V || splits < 1 || splits > 64 || (splits > 1 && !work))
    return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(sample_kernel, dim3(rows, splits), dim3(THREADS), 0, s, logits, ld, V, temperature,
                     top_k, top_p, u, u_step, u_stride, tokens, work);
  return kvf_last_error();
}

namespace {
// After a decode step of single tokens: the sampled token of every live sequence (context length
// above zero; padding sequences stay empty) becomes its next input, one position on, and is
// kept in row *counter of `ring` for the host, which reads all rows of a run of steps at once.
__global__ void decode_advance_kernel(const int* __restrict__ sampled, int* __restrict__ token_ids,
                                      int* __restrict__ positions, int* __restrict__ ctx_lens,
                                      int* __restrict__ ring, int* __restrict__ counter, int rows,
                                      int ring_stride, int ring_rows) {
  const int j = *counter;
  __syncthreads();  // every thread has read the counter before it moves
  for (int i = threadIdx.x; i < rows; i += blockDim.x) {
    const int t = sampled[i];
    if (j >= 0 && j < ring_rows) ring[j * ring_stride + i] = t;
    if (ctx_lens[i] > 0) {
      token_ids[i] = t;
      positions[i] += 1;
      ctx_lens[i] += 1;
    }
  }
  if (threadIdx.x == 0) *counter = j + 1;
}
}  // namespace

KVF_EXPORT int kvf_decode_advance(const int* sampled, int* token_ids, int* positions, int* ctx_lens,
                                  int* ring, int* counter, int rows, int ring_stride, int ring_rows,
                                  hipStream_t s) {
  if (rows <= 0) return 0;
  if (rows > ring_stride || ring_rows <= 0) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(decode_advance_kernel, dim3(1), dim3(256), 0, s, sampled, token_ids, positions,
                     ctx_lens, ring, counter, rows, ring_stride, ring_rows);
  return kvf_last_error();
}
