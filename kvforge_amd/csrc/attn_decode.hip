// Paged attention for single-token queries (decode), memory-bound: K and V of one kv head are
// streamed once and shared by the query heads of its group.
//
// Grid (decode sequence, kv head x head chunk, split of the key range).  In a wave, LPK lanes
// share one key: each loads 8 consecutive elements of the key's row (16 B for bf16) and the
// dot product is finished by a shuffle reduction over those lanes, so a wave handles
// 64 / LPK keys per iteration and the four waves of a workgroup take consecutive key groups.
// Every lane group keeps its own running maximum, sum and accumulator (fp32), rescaling only
// when the maximum grows; groups, waves and splits are merged at the end with the usual
// log-sum-exp rule.  With one split the output is written directly; otherwise partial
// (max, sum, accumulator) triples go to a workspace and a second small kernel merges them in
// split order.  (Merging in the workgroup that finishes last would save that launch, but the
// device-scope fences it needs write back the whole L2 and cost more than they save.)
//
// A window w > 0 restricts the keys to (p - w, p].  Pages are [num_blocks, KV, block_size, d].
#include "common.h"

namespace {
constexpr int WAVES = 4;

struct DecArgs {
  int H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs, splits;
  float scale;
};

// eight consecutive elements of a cache row, kept packed while their load is in flight
template <typename T> struct RawRow;
template <> struct RawRow<bf16_t> {
  typedef uint4 type;
  static __device__ __forceinline__ type zero() { return make_uint4(0u, 0u, 0u, 0u); }
  static __device__ __forceinline__ type load(const bf16_t* p) {
    return *reinterpret_cast<const uint4*>(p);
  }
  static __device__ __forceinline__ void unpack(const type& r, float (&v)[8]) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};
template <> struct RawRow<float> {
  struct type { float4 a, b; };
  static __device__ __forceinline__ type zero() {
    return type{make_float4(0.f, 0.f, 0.f, 0.f), make_float4(0.f, 0.f, 0.f, 0.f)};
  }
  static __device__ __forceinline__ type load(const float* p) {
    return type{*reinterpret_cast<const float4*>(p), *reinterpret_cast<const float4*>(p + 4)};
  }
  static __device__ __forceinline__ void unpack(const type& r, float (&v)[8]) {
    v[0] = r.a.x; v[1] = r.a.y; v[2] = r.a.z; v[3] = r.a.w;
    v[4] = r.b.x; v[5] = r.b.y; v[6] = r.b.z; v[7] = r.b.w;
  }
};

template <bool EXACT> __device__ __forceinline__ float exp_fn(float x) {
  return EXACT ? expf(x) : __expf(x);
}

template <typename T, int LPK, int GC, bool EXACT>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, T* __restrict__ out,
    float* __restrict__ part_acc, float* __restrict__ part_ml, DecArgs a) {
  constexpr int KPW = KVF_WAVE / LPK;  // keys per wave per iteration
  __shared__ float red_acc[WAVES][GC][LPK * 8];
  __shared__ float red_ml[WAVES][GC][2];

  const int seq = seq_ids ? seq_ids[blockIdx.x] : blockIdx.x;
  if (seq < 0 || seq >= a.n_seqs) return;
  const int G = a.H / a.KV, D = a.d;
  const int chunks = (G + GC - 1) / GC;
  const int kvh = blockIdx.y / chunks, g0 = (blockIdx.y - kvh * chunks) * GC;
  const int split = blockIdx.z;
  const int tok = cu_q[seq];
  const int ctx = ctx_lens[seq];
  const int pos = ctx - 1;
  int lo = 0;
  if (a.window > 0 && pos - a.window + 1 > 0) lo = pos - a.window + 1;
  // the key range [lo, ctx) is cut into `splits` runs of `per` keys, a multiple of the
  // workgroup's stride; runs past the end are empty and still take part in the merge
  const int nkeys = ctx > lo ? ctx - lo : 0;
  int per = (nkeys + a.splits - 1) / a.splits;
  per = (per + WAVES * KPW - 1) / (WAVES * KPW) * (WAVES * KPW);
  const int k_begin = lo + split * per;
  int k_end = k_begin + per;
  if (k_end > ctx) k_end = ctx;

  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int kg = lane / LPK, e0 = (lane % LPK) * 8;
  const bool lane_on = e0 < D;
  const int* table = block_table + static_cast<size_t>(seq) * a.table_stride;

  float qv[GC][8], acc[GC][8], m[GC], l[GC];
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { acc[g][e] = 0.f; qv[g][e] = 0.f; }
    if (lane_on && g0 + g < G)
      load8(q + static_cast<size_t>(tok) * a.q_stride + (kvh * G + g0 + g) * D + e0, qv[g]);
  }

  // Rounds of UNR keys per lane group.  The loads of round r + 1 (page ids first, then the K and
  // V rows they name) are issued before round r is consumed, so two rounds are in flight.
  constexpr int STRIDE = WAVES * KPW;
  constexpr int UNR = sizeof(T) == 2 ? 4 : 2;
  typedef typename RawRow<T>::type Raw;
  // two register buffers, named apart: an index chosen at run time would put them in scratch
  Raw kA[UNR], vA[UNR], kB[UNR], vB[UNR];
  bool okA[UNR], okB[UNR];
  const int j_first = k_begin + wave * KPW + kg;

  auto issue = [&](int j0, Raw (&kb)[UNR], Raw (&vb)[UNR], bool (&okb)[UNR]) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int j = j0 + u * STRIDE;
      bool ok = false;
      size_t base = 0;
      if (j < k_end) {
        const int blk = j / a.block_size;
        const int page = blk < a.table_stride ? table[blk] : -1;
        ok = page >= 0 && page < a.num_blocks;
        base = ((static_cast<size_t>(ok ? page : 0) * a.KV + kvh) * a.block_size +
                (j - blk * a.block_size)) * D + e0;
      }
      okb[u] = ok;
      kb[u] = RawRow<T>::zero();
      vb[u] = RawRow<T>::zero();
      if (ok && lane_on) {
        kb[u] = RawRow<T>::load(k_pages + base);
        vb[u] = RawRow<T>::load(v_pages + base);
      }
    }
  };
  auto consume = [&](const Raw (&kb)[UNR], const Raw (&vb)[UNR], const bool (&okb)[UNR]) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      float kf[8], vf[8];
      RawRow<T>::unpack(kb[u], kf);
      RawRow<T>::unpack(vb[u], vf);
#pragma unroll
      for (int g = 0; g < GC; ++g) {
        if (g0 + g >= G) break;
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s = fmaf(qv[g][e], kf[e], s);
        s = group_sum<LPK>(s);
        if (!okb[u]) continue;
        s *= a.scale;
        if (s > m[g]) {
          const float c = exp_fn<EXACT>(m[g] - s);
          l[g] *= c;
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] *= c;
          m[g] = s;
        }
        const float p = exp_fn<EXACT>(s - m[g]);
        l[g] += p;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(p, vf[e], acc[g][e]);
      }
    }
  };
  // every lane group of the workgroup runs the same number of rounds (shuffles stay converged)
  const int rounds = (k_end - k_begin + UNR * STRIDE - 1) / (UNR * STRIDE);
  constexpr int RSTEP = UNR * STRIDE;
  if (rounds > 0) issue(j_first, kA, vA, okA);
  for (int r = 0; r < rounds; r += 2) {
    if (r + 1 < rounds) issue(j_first + (r + 1) * RSTEP, kB, vB, okB);
    consume(kA, vA, okA);
    if (r + 1 < rounds) {
      if (r + 2 < rounds) issue(j_first + (r + 2) * RSTEP, kA, vA, okA);
      consume(kB, vB, okB);
    }
  }

  // merge the key groups of a wave (lanes that hold the same elements: xor LPK, 2*LPK, ...)
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    float mm = m[g];
#pragma unroll
    for (int o = LPK; o < KVF_WAVE; o <<= 1) mm = fmaxf(mm, __shfl_xor(mm, o, KVF_WAVE));
    const float c = (m[g] == -INFINITY) ? 0.f : exp_fn<EXACT>(m[g] - mm);
    float ll = l[g] * c;
#pragma unroll
    for (int o = LPK; o < KVF_WAVE; o <<= 1) ll += __shfl_xor(ll, o, KVF_WAVE);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float v = acc[g][e] * c;
#pragma unroll
      for (int o = LPK; o < KVF_WAVE; o <<= 1) v += __shfl_xor(v, o, KVF_WAVE);
      acc[g][e] = v;
    }
    if (kg == 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) red_acc[wave][g][e0 + e] = acc[g][e];
      if (lane == 0) { red_ml[wave][g][0] = mm; red_ml[wave][g][1] = ll; }
    }
  }
  __syncthreads();
  // merge the waves: thread t -> (head g, element e)
  for (int idx = threadIdx.x; idx < GC * LPK * 8; idx += 256) {
    const int g = idx / (LPK * 8), e = idx - g * (LPK * 8);
    if (g0 + g >= G || e >= D) continue;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, red_ml[w][g][0]);
    float ll = 0.f, v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float mw = red_ml[w][g][0];
      const float c = (mw == -INFINITY) ? 0.f : exp_fn<EXACT>(mw - mm);
      ll += red_ml[w][g][1] * c;
      v += red_acc[w][g][e] * c;
    }
    const int head = kvh * G + g0 + g;
    if (a.splits == 1) {
      Elem<T>::store(out + static_cast<size_t>(tok) * a.o_stride + head * D + e,
                     ll > 0.f ? v / ll : 0.f);
    } else {
      const size_t slot = (static_cast<size_t>(blockIdx.x) * a.H + head) * a.splits + split;
      part_acc[slot * D + e] = v;
      if (e == 0) { part_ml[slot * 2] = mm; part_ml[slot * 2 + 1] = ll; }
    }
  }
}

// Merges the splits of every (sequence, head) in split order.
template <typename T, bool EXACT>
__global__ void attn_decode_combine_kernel(const float* __restrict__ part_acc,
                                           const float* __restrict__ part_ml,
                                           const int* __restrict__ seq_ids,
                                           const int* __restrict__ cu_q, T* __restrict__ out,
                                           int H, int D, int splits, int o_stride, int n_seqs) {
  const int seq = seq_ids ? seq_ids[blockIdx.x] : blockIdx.x;
  if (seq < 0 || seq >= n_seqs) return;
  const int head = blockIdx.y;
  const size_t slot0 = (static_cast<size_t>(blockIdx.x) * H + head) * splits;
  float mm = -INFINITY;
  for (int s = 0; s < splits; ++s) mm = fmaxf(mm, part_ml[(slot0 + s) * 2]);
  const int tok = cu_q[seq];
  for (int e = threadIdx.x; e < D; e += blockDim.x) {
    float ll = 0.f, v = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float ms = part_ml[(slot0 + s) * 2];
      const float c = (ms == -INFINITY) ? 0.f : exp_fn<EXACT>(ms - mm);
      ll += part_ml[(slot0 + s) * 2 + 1] * c;
      v += part_acc[(slot0 + s) * D + e] * c;
    }
    Elem<T>::store(out + static_cast<size_t>(tok) * o_stride + head * D + e,
                   ll > 0.f ? v / ll : 0.f);
  }
}

template <typename T, bool EXACT>
int launch(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
           const int* seq_ids, const int* cu_q, const int* ctx_lens, void* out, float* part_acc,
           float* part_ml, int num_seqs, DecArgs a, hipStream_t s) {
  if (num_seqs <= 0) return 0;
  const int G = a.H / a.KV;
  const int lanes = a.d / 8 + (a.d % 8 ? 1 : 0);
  const int lpk = lanes <= 2 ? 2 : lanes <= 4 ? 4 : lanes <= 8 ? 8 : lanes <= 16 ? 16 : 32;
  const int gc = G <= 4 ? 4 : 8;
  const int chunks = (G + gc - 1) / gc;
  dim3 grid(num_seqs, a.KV * chunks, a.splits);
#define GO(LPK, GC)                                                                               \
  hipLaunchKernelGGL((attn_decode_kernel<T, LPK, GC, EXACT>), grid, dim3(256), 0, s,              \
                     static_cast<const T*>(q), static_cast<const T*>(k_pages),                    \
                     static_cast<const T*>(v_pages), block_table, seq_ids, cu_q, ctx_lens,        \
                     static_cast<T*>(out), part_acc, part_ml, a)
#define PICK(GC)                                                                                  \
  switch (lpk) {                                                                                  \
    case 2: GO(2, GC); break;                                                                     \
    case 4: GO(4, GC); break;                                                                     \
    case 8: GO(8, GC); break;                                                                     \
    case 16: GO(16, GC); break;                                                                   \
    default: GO(32, GC); break;                                                                   \
  }
  if (gc == 4) { PICK(4) } else { PICK(8) }
#undef PICK
#undef GO
  int err = kvf_last_error();
  if (err || a.splits == 1) return err;
  hipLaunchKernelGGL((attn_decode_combine_kernel<T, EXACT>), dim3(num_seqs, a.H), dim3(64), 0, s,
                     part_acc, part_ml, seq_ids, cu_q, static_cast<T*>(out), a.H, a.d, a.splits,
                     a.o_stride, a.n_seqs);
  return kvf_last_error();
}
}  // namespace

// dtype: 0 = fp32 (accurate exp), 1 = bf16.  d: multiple of 16, at most 256.
// With splits > 1, part_acc holds num_seqs*H*splits*d floats and part_ml num_seqs*H*splits*2;
// calls that share these buffers must not overlap.
KVF_EXPORT int kvf_attn_decode(int dtype, const void* q, const void* k_pages, const void* v_pages,
                               const int* block_table, const int* seq_ids, const int* cu_q,
                               const int* ctx_lens, void* out, float* part_acc, float* part_ml,
                               int num_seqs, int H, int KV, int d, int block_size, int num_blocks,
                               int table_stride, int q_stride, int o_stride, int window,
                               int n_seqs, int splits, float scale, hipStream_t s) {
  if (d % 16 != 0 || d > 256 || d <= 0 || KV <= 0 || H % KV != 0 || splits < 1)
    return static_cast<int>(hipErrorInvalidValue);
  if (splits > 1 && (!part_acc || !part_ml)) return static_cast<int>(hipErrorInvalidValue);
  DecArgs a{H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs,
            splits, scale};
  if (dtype == 0)
    return launch<float, true>(q, k_pages, v_pages, block_table, seq_ids, cu_q, ctx_lens, out,
                               part_acc, part_ml, num_seqs, a, s);
  if (dtype == 1)
    return launch<bf16_t, false>(q, k_pages, v_pages, block_table, seq_ids, cu_q, ctx_lens, out,
                                 part_acc, part_ml, num_seqs, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}
