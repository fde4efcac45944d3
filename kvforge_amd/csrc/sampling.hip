// Token selection from fp32 logits, one workgroup of 16 waves per row (several for greedy rows).
//
//   temperature == 0      : argmax, the lowest index among equal maxima.
//   temperature  > 0      : z = logits / temperature; optional top-k, then optional top-p on the
//                           renormalised top-k set; p = softmax over what is kept (fp32);
//                           the token is the first index, in vocabulary order, whose cumulative
//                           probability exceeds u * total, u in [0, 1) given by the caller.
// top-k keeps every value >= the k-th largest (equal values are kept together); top-p keeps a
// value iff the mass of strictly larger kept values is below top_p, so the largest is always kept.
// Both thresholds are found digit by digit over the order-preserving integer image of a float
// (three passes over the row each, weights summed per digit in LDS), which needs no sort and no
// memory beyond the row itself.
#include "common.h"
#include "sampling_static.h"

#include <cstdio>
#include <mutex>

namespace {
constexpr int THREADS = 1024, NWAVES = THREADS / KVF_WAVE;

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// exp(s - max) through the hardware's base-2 exponential: the argument is at most 0, the result
// in (0, 1] with a relative error of a few 2^-24 (the full-precision routine is ten times the
// instructions and was most of the kernel's time)
__device__ __forceinline__ float mass_of(float s, float mx) {
  return __builtin_amdgcn_exp2f((s - mx) * 1.44269504088896340736f);
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

// f(i, x[i]) for every element of a row, each thread with eight 16-byte loads in flight where the
// row starts on 16 bytes (element by element otherwise).
template <typename F>
__device__ __forceinline__ void each_logit(const float* __restrict__ x, int V, F f) {
  constexpr int U = 8;
  const int tid = threadIdx.x;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
  const int v4 = vec ? V / 4 : 0;
  const float4* x4 = reinterpret_cast<const float4*>(x);
  for (int i0 = tid; i0 < v4; i0 += U * THREADS) {
    float4 r[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i0 + u * THREADS < v4) r[u] = x4[i0 + u * THREADS];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (i0 + u * THREADS >= v4) break;
      const int base = 4 * (i0 + u * THREADS);
      f(base, r[u].x);
      f(base + 1, r[u].y);
      f(base + 2, r[u].z);
      f(base + 3, r[u].w);
    }
  }
  for (int i = 4 * v4 + tid; i < V; i += THREADS) f(i, x[i]);
}

// Threshold search for top-k and top-p without a sort and without 32 passes of bisection: the
// order-preserving key is settled 11, 11 and 10 bits at a time.  A pass adds every candidate's
// weight (1 for top-k; its share of the probability mass as a 40-bit fixed-point number for
// top-p) to the bin of its next digit in LDS; integer sums do not depend on the order of the
// additions, so the result is reproducible.  Walking the bins from the top, the digit is the
// first bin at which the weight accumulated so far (the bin's own included) reaches the target:
// the k-th largest value for a target of k, and for top-p the smallest value that is still kept
// (the weight of all strictly larger values is below the target, and no longer so after it).
constexpr int RADIX_BINS = 2048;
constexpr float MASS_ONE = 1099511627776.f;  // 2^40

template <bool MASS>
__device__ uint32_t radix_threshold(const float* __restrict__ x, int V, float inv_t, float mx,
                                    uint32_t floor_key, float pp, int k,
                                    unsigned long long* hist, unsigned long long* pick) {
  const int tid = threadIdx.x, lane = tid % KVF_WAVE;
  uint32_t prefix = 0;
  int settled = 0;
  unsigned long long above = 0, target = MASS ? 0ull : static_cast<unsigned long long>(k);
#pragma unroll 1
  for (int level = 0; level < 3; ++level) {
    const int bits = level == 2 ? 10 : 11;
    const int shift = 32 - settled - bits;
    for (int b = tid; b < RADIX_BINS; b += THREADS) hist[b] = 0ull;
    __syncthreads();
    each_logit(x, V, [&](int, float v) {
      const float sc = v * inv_t;
      const uint32_t key = order_key(sc);
      if (key < floor_key) return;
      if (settled && (key >> (32 - settled)) != prefix) return;
      const unsigned long long w =
          MASS ? static_cast<unsigned long long>(mass_of(sc, mx) * MASS_ONE) : 1ull;
      if (w) atomicAdd(hist + ((key >> shift) & ((1u << bits) - 1u)), w);
    });
    __syncthreads();
    if (tid < KVF_WAVE) {
      // lane l owns the 32 bins from 2047 - 32 l downwards
      const int nb = 1 << bits, per = RADIX_BINS / KVF_WAVE, top = nb - 1 - lane * per;
      unsigned long long mine = 0;
      for (int j = 0; j < per; ++j)
        if (top - j >= 0) mine += hist[top - j];
      unsigned long long incl = mine;  // sum over lanes 0..l
#pragma unroll
      for (int o = 1; o < KVF_WAVE; o <<= 1) {
        const unsigned long long n = __shfl_up(incl, o, KVF_WAVE);
        if (lane >= o) incl += n;
      }
      if (MASS && level == 0) {
        const unsigned long long total = __shfl(incl, KVF_WAVE - 1, KVF_WAVE);
        target = static_cast<unsigned long long>(static_cast<double>(pp) * static_cast<double>(total));
      }
      const unsigned long long want = target > above ? target - above : 0ull;
      const unsigned long long need = want > 1ull ? want : 1ull;  // an empty bin never counts
      const unsigned long long hits = __ballot(incl >= need);
      // no bin reaches the target (rounding): everything is kept, down to the lowest weight
      const int owner = hits ? __ffsll(static_cast<long long>(hits)) - 1
                             : 63 - __clzll(static_cast<long long>(__ballot(mine > 0ull) | 1ull));
      if (lane == owner) {
        unsigned long long run = incl - mine;
        int chosen = -1, last = -1;
        for (int j = 0; j < per && chosen < 0; ++j) {
          const int b = top - j;
          if (b < 0) break;
          const unsigned long long h = hist[b];
          if (h) last = b;
          if (h && run + h >= need) { chosen = b; break; }
          run += h;
        }
        if (chosen < 0) {                 // only without a hit: the lowest bin that holds weight
          chosen = last < 0 ? 0 : last;
          run -= hist[chosen];
        }
        pick[0] = static_cast<unsigned long long>(chosen);
        pick[1] = above + run;
      }
    }
    __syncthreads();
    prefix = (prefix << bits) | static_cast<uint32_t>(pick[0]);
    above = pick[1];
    settled += bits;
    __syncthreads();
  }
  return prefix;
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
  __shared__ int sh_idx[NWAVES];
  __shared__ unsigned long long hist[RADIX_BINS];
  __shared__ unsigned long long pick[2];
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
  each_logit(x, V, [&](int, float v) { mx = fmaxf(mx, v * inv_t); });
  mx = block_reduce_max(mx, sh);

  // ---- top-k: key of the k-th largest value (0 keeps everything)
  uint32_t key_min = 0;
  const int k = top_k ? top_k[row] : 0;
  if (k > 0 && k < V) key_min = radix_threshold<false>(x, V, inv_t, mx, 0u, 1.f, k, hist, pick);
  // ---- top-p on the top-k set: the smallest value whose strictly larger values weigh less than
  // top_p of the set
  const float pp = top_p ? top_p[row] : 1.f;
  if (pp < 1.f) {
    const uint32_t v = radix_threshold<true>(x, V, inv_t, mx, key_min, pp > 0.f ? pp : 0.f, 0, hist, pick);
    if (v > key_min) key_min = v;
  }

  // ---- inverse CDF in vocabulary order.  The row is cut into chunks of `chunk` consecutive
  // elements (256, or a multiple for very large vocabularies); the waves take chunks in turn and
  // leave each chunk's mass in LDS; wave 0 finds the chunk that holds u * total and walks it.
  float* chunk_sum = reinterpret_cast<float*>(hist);  // the bins are not needed any more
  constexpr int MAX_CHUNKS = 1024, LANE_ELEMS = 4;
  const int per_iter = KVF_WAVE * LANE_ELEMS;
  const int chunk = per_iter * ((V + per_iter * MAX_CHUNKS - 1) / (per_iter * MAX_CHUNKS));
  const int n_chunks = (V + chunk - 1) / chunk;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
  auto lane_mass = [&](int first, float (&p)[LANE_ELEMS]) {
    // the kept mass of elements first .. first+3 (those past V are nothing)
    float v[LANE_ELEMS] = {0.f, 0.f, 0.f, 0.f};
    if (vec && first + LANE_ELEMS <= V) {
      const float4 r = *reinterpret_cast<const float4*>(x + first);
      v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
    } else {
#pragma unroll
      for (int e = 0; e < LANE_ELEMS; ++e)
        if (first + e < V) v[e] = x[first + e];
    }
#pragma unroll
    for (int e = 0; e < LANE_ELEMS; ++e) {
      const float sc = v[e] * inv_t;
      p[e] = first + e < V && order_key(sc) >= key_min ? mass_of(sc, mx) : 0.f;
    }
  };
  // four chunks of a wave at a time, so that their loads are in flight together
  for (int c0 = wave; c0 < n_chunks; c0 += 4 * NWAVES) {
    float part[4] = {0.f, 0.f, 0.f, 0.f};
    for (int off = lane * LANE_ELEMS; off < chunk; off += per_iter) {
      float p[4][LANE_ELEMS];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int c = c0 + q * NWAVES;
        // a chunk past the end starts past V: its elements are nothing
        lane_mass(c < n_chunks ? c * chunk + off : V, p[q]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) part[q] += (p[q][0] + p[q][1]) + (p[q][2] + p[q][3]);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float sum = wave_sum(part[q]);
      if (lane == 0 && c0 + q * NWAVES < n_chunks) chunk_sum[c0 + q * NWAVES] = sum;
    }
  }
  __syncthreads();
  if (wave == 0) {
    // lane l owns chunks 16 l .. 16 l + 15
    constexpr int PER_LANE = MAX_CHUNKS / KVF_WAVE;
    float mine = 0.f;
    for (int j = 0; j < PER_LANE; ++j) {
      const int c = lane * PER_LANE + j;
      if (c < n_chunks) mine += chunk_sum[c];
    }
    float incl = mine;
#pragma unroll
    for (int o = 1; o < KVF_WAVE; o <<= 1) {
      const float nb = __shfl_up(incl, o, KVF_WAVE);
      if (lane >= o) incl += nb;
    }
    const float total = __shfl(incl, KVF_WAVE - 1, KVF_WAVE);
    const float target = u[(u_step ? *u_step * u_stride : 0) + row] * total;
    // the first lane, then the first of its chunks, whose mass carries the sum past the target
    const unsigned long long over = __ballot(mine > 0.f && incl > target);
    const unsigned long long any = __ballot(mine > 0.f);
    int found = -1;
    if (any) {
      // rounding may leave the target at or past the total: then the last lane with mass
      const int owner = over ? __ffsll(static_cast<long long>(over)) - 1 : 63 - __clzll(static_cast<long long>(any));
      float before = __shfl(incl - mine, owner, KVF_WAVE);
      int c_hit = -1, c_last = -1;
      for (int j = 0; j < PER_LANE; ++j) {   // the same in all lanes
        const int c = owner * PER_LANE + j;
        if (c >= n_chunks) break;
        const float m = chunk_sum[c];
        if (m > 0.f) c_last = c;
        if (m > 0.f && before + m > target) { c_hit = c; break; }
        before += m;
      }
      if (c_hit < 0) {           // the overshoot case: the last chunk with mass, from its start
        c_hit = c_last;
        before = -INFINITY;      // whatever is kept last in it is taken
      }
      float running = before;
      int last_kept = -1;
      for (int first = c_hit * chunk + lane * LANE_ELEMS; first - lane * LANE_ELEMS < min(V, (c_hit + 1) * chunk) && found < 0;
           first += per_iter) {
        float p[LANE_ELEMS];
        lane_mass(first, p);
        const float lane_total = (p[0] + p[1]) + (p[2] + p[3]);
        float lincl = lane_total;
#pragma unroll
        for (int o = 1; o < KVF_WAVE; o <<= 1) {
          const float nb = __shfl_up(lincl, o, KVF_WAVE);
          if (lane >= o) lincl += nb;
        }
        // within the lane: the first element that carries the sum past the target
        float acc = running + (lincl - lane_total);
        int hit_e = -1, kept_e = -1;
#pragma unroll
        for (int e = 0; e < LANE_ELEMS; ++e) {
          if (p[e] > 0.f) {
            kept_e = e;
            if (hit_e < 0 && acc + p[e] > target) hit_e = e;
          }
          acc += p[e];
        }
        const unsigned long long hits = __ballot(hit_e >= 0);
        const unsigned long long kept = __ballot(kept_e >= 0);
        if (hits) {
          const int src = __ffsll(static_cast<long long>(hits)) - 1;
          found = __shfl(first + hit_e, src, KVF_WAVE);
        }
        if (kept) {
          const int src = 63 - __clzll(static_cast<long long>(kept));
          last_kept = __shfl(first + kept_e, src, KVF_WAVE);
        }
        running += __shfl(lincl, KVF_WAVE - 1, KVF_WAVE);
      }
      if (found < 0) found = last_kept;
    }
    if (lane == 0) tokens[row] = found >= 0 ? found : 0;
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
// Work memory of kvf_sample_static: tickets, then the chunks' best values, then their indices.
// The array is part of the library's image, so every GPU the library runs on holds a copy at an
// address of its own.  In host code the name below only stands for the symbol; the device
// address comes from hipGetSymbolAddress and is what launches are given.
static __device__ __align__(256) int scratch[KVF_SAMPLE_STATIC_MAX_ROWS * (1 + 2 * KVF_SAMPLE_STATIC_MAX_SPLITS)];
constexpr int MAX_DEVICES = 64;
int* scratch_address[MAX_DEVICES];  // per device, looked up at the first call on it
std::mutex scratch_lock;

__global__ void clear_ints_kernel(int* __restrict__ p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// Compute units of the current device, asked of the runtime once per device; 0 if it does not say.
int compute_units_of_current_device() {
  static int units[MAX_DEVICES];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 0;
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (units[dev] <= 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    units[dev] = n;
  }
  return units[dev];
}

// The device address of `scratch` on the current device; null (and *code set) if the runtime
// does not give it.
int* scratch_on_current_device(hipError_t* code) {
  int dev = -1;
  *code = hipGetDevice(&dev);
  if (*code != hipSuccess) return nullptr;
  if (dev < 0 || dev >= MAX_DEVICES) {
    *code = hipErrorInvalidDevice;
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (!scratch_address[dev]) {
    void* p = nullptr;
    *code = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (*code != hipSuccess || !p) {
      if (*code == hipSuccess) *code = hipErrorInvalidSymbol;
      return nullptr;
    }
    scratch_address[dev] = static_cast<int*>(p);
  }
  return scratch_address[dev];
}
}  // namespace

KVF_EXPORT int kvf_sample_static(const float* logits, int ld, int rows, int V, const float* temperature,
                                 const int* top_k, const float* top_p, const float* u,
                                 const int* u_step, int u_stride, int* tokens, hipStream_t s) {
  if (rows <= 0) return 0;
  if (rows > KVF_SAMPLE_STATIC_MAX_ROWS) {
    fprintf(stderr, "kvf_sample_static: %d rows asked for, at most %d fit its work memory\n", rows,
            KVF_SAMPLE_STATIC_MAX_ROWS);
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (V <= 0 || ld < V) return static_cast<int>(hipErrorInvalidValue);
  // about one workgroup per compute unit, each with at least 4096 logits
  int splits = KVF_SAMPLE_STATIC_MAX_SPLITS;
  const int units = compute_units_of_current_device();
  if (units <= 0) return static_cast<int>(hipErrorInvalidDevice);
  if (splits > units / rows) splits = units / rows;
  if (splits > V / 4096) splits = V / 4096;
  if (splits < 1) splits = 1;
  int* work = nullptr;
  if (splits > 1) {
    hipError_t code = hipSuccess;
    work = scratch_on_current_device(&code);
    if (!work) return static_cast<int>(code);
    // the tickets start at zero whatever the call before left (a fill kernel, not a memset
    // node: the launches may be captured)
    hipLaunchKernelGGL(clear_ints_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, work, rows);
    const int launched = kvf_last_error();
    if (launched != 0) return launched;
  }
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
