// Paged attention of the true 32-bit path: every product and sum in fp32.  It takes bf16
// operands as well (widened exactly), for caches whose pages the bf16 kernels do not take.
//
// Query runs of any length (attn_mfma32_kernel): fp32 on the matrix cores with
// v_mfma_f32_16x16x4_f32, which multiplies and adds in fp32.  Row r of a sequence is
// (query token r / G, head r % G of the kv head's group), so the G query heads that share a kv
// head also share every K/V tile.  A workgroup of four waves takes an item of 64 rows of one
// (sequence, kv head), a wave 16 of them.  Keys are walked in tiles aligned to multiples of the
// tile size from position 0; the tile's keys, then its values, are staged in LDS for the four
// waves.  A wave computes the transposed scores S^T = K Q^T (keys down the instruction's rows),
// so that a lane ends up with four neighbouring keys of one query row: the running maximum and
// sum of a row are a lane's own, the probabilities stay in registers and are the right-hand
// operand of O^T += V^T P as they are.  Key j is visible to the query at position p iff j <= p,
// j < context length and, with a window w > 0, j > p - w.  Scores are scaled after the dot
// product; with `slopes` (one number per q head) slopes[h] * (j - p) is added to them, a bias by
// distance.  The order of every sum is fixed by the positions alone.
//
// K pages are [num_blocks, KV, block_size, d], V pages are transposed [num_blocks, KV, d,
// block_size]; a key whose page entry is negative or out of range reads as zeros.
#include "common.h"

namespace {
constexpr int ITEM_ROWS = 64;   // rows per work item: four waves of 16

struct AttnArgs {
  int H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs;
  float scale;
  const float* slopes;  // null, or one number per q head: slopes[h] * (key - query position) is added to a score
};

typedef float f32x4 __attribute__((ext_vector_type(4)));

// four consecutive elements as floats; p on 16 bytes (fp32) / 8 bytes (bf16)
__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4(const bf16_t* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return f32x4{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
               __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u)};
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, f32x4 v) {
  uint2 r;
  r.x = static_cast<uint32_t>(f32_to_bf16(v[0])) | (static_cast<uint32_t>(f32_to_bf16(v[1])) << 16);
  r.y = static_cast<uint32_t>(f32_to_bf16(v[2])) | (static_cast<uint32_t>(f32_to_bf16(v[3])) << 16);
  *reinterpret_cast<uint2*>(p) = r;
}

// The instruction: D[i][j] += sum_k A[i][k] B[k][j] over k = 0..3; lane l gives A[l % 16][l / 16]
// and B[l / 16][l % 16] and holds D[4 (l / 16) + v][l % 16], v = 0..3.  Here the four lane
// groups stand for four *neighbouring* k each (group g takes k = 4 g + e in instruction e of
// four), so that a lane's operands are 16 consecutive bytes.
__device__ __forceinline__ f32x4 mfma4(float a, float b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

template <typename T, int DMAX>
__global__ __launch_bounds__(256) void attn_mfma32_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens, const int* __restrict__ work, T* __restrict__ out,
    AttnArgs a) {
  constexpr int DT = DMAX / 16;                // 16-element tiles of the head
  constexpr int BK = DMAX > 128 ? 32 : 64;     // keys per tile
  constexpr int ST = BK / 16;                  // 16-key blocks per tile
  constexpr int KLD = DMAX + 4, VLD = BK + 4;  // LDS rows 16 bytes apart in the banks
  constexpr int FLOATS = BK * KLD > DMAX * VLD ? BK * KLD : DMAX * VLD;
  __shared__ __align__(16) float KVs[FLOATS];  // the tile's keys [BK][KLD], then its values [d][VLD]

  // rows (sequence, item, item or -1): two workgroups per row, one for each item
  const int w = blockIdx.x >> 1;
  const int seq = work[3 * w];
  const int item = work[3 * w + 1 + (blockIdx.x & 1)];
  if (item < 0 || seq < 0 || seq >= a.n_seqs) return;
  const int kvh = blockIdx.y;
  const int G = a.H / a.KV, D = a.d;
  const int q0 = cu_q[seq], qlen = cu_q[seq + 1] - q0, ctx = ctx_lens[seq];
  const int start = ctx - qlen;  // position of the run's first query
  const int rows_total = qlen * G, item0 = item * ITEM_ROWS;
  if (item0 >= rows_total || qlen <= 0 || start < 0) return;

  const int tid = threadIdx.x, lane = tid % KVF_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / KVF_WAVE);
  const int j16 = lane % 16, g4 = lane / 16;
  const int* table = block_table + static_cast<size_t>(seq) * a.table_stride;

  // this lane's query row (the same in the four lane groups)
  const int r0 = item0 + wave * 16;
  const int row = r0 + j16;
  const bool row_ok = row < rows_total;
  const int tok = row_ok ? row / G : 0;
  const int head = kvh * G + (row_ok ? row - tok * G : 0);
  const int pos = start + tok;
  const float slope = a.slopes && row_ok ? a.slopes[head] : 0.f;
  // key ranges: of the workgroup's rows (what is staged) and of this wave's (what it works on)
  int last = item0 + ITEM_ROWS - 1;
  if (last >= rows_total) last = rows_total - 1;
  const int hi = min(start + last / G, ctx - 1);
  int lo = 0;
  if (a.window > 0) lo = max(0, start + item0 / G - a.window + 1);
  int hi_w = -1, lo_w = 0;
  if (r0 < rows_total) {
    int last_w = r0 + 15;
    if (last_w >= rows_total) last_w = rows_total - 1;
    hi_w = min(start + last_w / G, ctx - 1);
    if (a.window > 0) lo_w = max(0, start + r0 / G - a.window + 1);
  }

  // the query row's elements 16 u + 4 g4 .. + 3, u = 0 .. DT - 1
  f32x4 qf[DT];
  {
    const T* qp = q + static_cast<size_t>(q0 + tok) * a.q_stride + head * D + 4 * g4;
#pragma unroll
    for (int u = 0; u < DT; ++u)
      qf[u] = (row_ok && 16 * u < D) ? load4(qp + 16 * u) : f32x4{0.f, 0.f, 0.f, 0.f};
  }

  float m_run = -INFINITY, l_run = 0.f;
  f32x4 acc[DT];   // acc[t][v]: element 16 t + 4 g4 + v of this lane's row
#pragma unroll
  for (int t = 0; t < DT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bool quads = a.block_size % 4 == 0;
  const int chunks = D / 8;
  for (int t0 = (lo / BK) * BK; t0 <= hi; t0 += BK) {
    // ---- keys of the tile
    __syncthreads();   // the values of the tile before have been used
    for (int ch = tid; ch < BK * chunks; ch += 256) {
      const int c = ch / chunks, k8 = (ch - c * chunks) * 8;
      const int j = t0 + c;
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (j >= lo && j <= hi) {
        const int blk = j / a.block_size;
        const int page = blk < a.table_stride ? table[blk] : -1;
        if (page >= 0 && page < a.num_blocks)
          load8(k_pages + ((static_cast<size_t>(page) * a.KV + kvh) * a.block_size +
                           (j - blk * a.block_size)) * D + k8, v);
      }
      *reinterpret_cast<float4*>(&KVs[c * KLD + k8]) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(&KVs[c * KLD + k8 + 4]) = make_float4(v[4], v[5], v[6], v[7]);
    }
    __syncthreads();
    const bool mine = t0 <= hi_w && t0 + BK > lo_w;   // the same in all lanes of the wave
    f32x4 p[ST];
    float corr = 1.f;
    if (mine) {
      // ---- transposed scores: p[st][v] = key t0 + 16 st + 4 g4 + v against this lane's row
      float tmax = -INFINITY;
#pragma unroll
      for (int st = 0; st < ST; ++st) {
        f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < DT; ++u) {
          if (16 * u >= D) break;
          const f32x4 kf = *reinterpret_cast<const f32x4*>(&KVs[(16 * st + j16) * KLD + 16 * u + 4 * g4]);
#pragma unroll
          for (int e = 0; e < 4; ++e) sc = mfma4(kf[e], qf[u][e], sc);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int j = t0 + 16 * st + 4 * g4 + v;
          bool vis = row_ok && j <= pos && j < ctx;
          if (a.window > 0) vis = vis && (j > pos - a.window);
          sc[v] = vis ? fmaf(slope, static_cast<float>(j - pos), sc[v] * a.scale) : -INFINITY;
          tmax = fmaxf(tmax, sc[v]);
        }
        p[st] = sc;
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, KVF_WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, KVF_WAVE));
      const float m_new = fmaxf(m_run, tmax);
      float psum = 0.f;
      if (m_new == -INFINITY) {
#pragma unroll
        for (int st = 0; st < ST; ++st) p[st] = f32x4{0.f, 0.f, 0.f, 0.f};
      } else {
        corr = expf(m_run - m_new);  // exp(-inf) = 0 on the first visible tile
#pragma unroll
        for (int st = 0; st < ST; ++st)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float e = expf(p[st][v] - m_new);
            p[st][v] = e;
            psum += e;
          }
      }
      psum += __shfl_xor(psum, 16, KVF_WAVE);
      psum += __shfl_xor(psum, 32, KVF_WAVE);
      l_run = l_run * corr + psum;
      m_run = m_new;
    }
    // ---- values of the tile (over the keys, once every wave has finished with them)
    __syncthreads();
    if (quads) {
      // four neighbouring keys of one element lie side by side in a page
      for (int idx = tid; idx < D * (BK / 4); idx += 256) {
        const int e = idx / (BK / 4), c = (idx - e * (BK / 4)) * 4;
        const int j = t0 + c;
        f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
        if (j + 3 >= lo && j <= hi) {
          const int blk = j / a.block_size;
          const int page = blk < a.table_stride ? table[blk] : -1;
          if (page >= 0 && page < a.num_blocks) {
            v = load4(v_pages + ((static_cast<size_t>(page) * a.KV + kvh) * D + e) * a.block_size +
                      (j - blk * a.block_size));
#pragma unroll
            for (int x = 0; x < 4; ++x)
              if (j + x < lo || j + x > hi) v[x] = 0.f;
          }
        }
        *reinterpret_cast<f32x4*>(&KVs[e * VLD + c]) = v;
      }
    } else {
      for (int idx = tid; idx < BK * D; idx += 256) {
        const int e = idx / BK, c = idx - e * BK;
        const int j = t0 + c;
        float v = 0.f;
        if (j >= lo && j <= hi) {
          const int blk = j / a.block_size;
          const int page = blk < a.table_stride ? table[blk] : -1;
          if (page >= 0 && page < a.num_blocks)
            v = Elem<T>::load(v_pages + ((static_cast<size_t>(page) * a.KV + kvh) * D + e) * a.block_size +
                              (j - blk * a.block_size));
        }
        KVs[e * VLD + c] = v;
      }
    }
    __syncthreads();
    if (mine) {
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        if (16 * t >= D) break;
        f32x4 o = acc[t] * corr;
#pragma unroll
        for (int st = 0; st < ST; ++st) {
          const f32x4 vf = *reinterpret_cast<const f32x4*>(&KVs[(16 * t + j16) * VLD + 16 * st + 4 * g4]);
#pragma unroll
          for (int v = 0; v < 4; ++v) o = mfma4(vf[v], p[st][v], o);
        }
        acc[t] = o;
      }
    }
  }
  if (!row_ok) return;
  T* o = out + static_cast<size_t>(q0 + tok) * a.o_stride + head * D + 4 * g4;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
  for (int t = 0; t < DT; ++t)
    if (16 * t < D) store4(o + 16 * t, acc[t] * inv);
}

template <typename T>
int launch(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
           const int* cu_q, const int* ctx_lens, const int* work, int num_work, void* out,
           AttnArgs a, hipStream_t s) {
  if (num_work <= 0) return 0;
  dim3 grid(2 * num_work, a.KV);
#define GO(DMAX)                                                                                  \
  hipLaunchKernelGGL((attn_mfma32_kernel<T, DMAX>), grid, dim3(256), 0, s,                        \
                     static_cast<const T*>(q), static_cast<const T*>(k_pages),                    \
                     static_cast<const T*>(v_pages), block_table, cu_q, ctx_lens, work,           \
                     static_cast<T*>(out), a)
  if (a.d <= 64) GO(64);
  else if (a.d <= 128) GO(128);
  else GO(256);
#undef GO
  return kvf_last_error();
}

// ---------------------------------------------------------------------------------------------
// Single-token queries (decode steps).  A workgroup of four waves takes one (sequence, kv head,
// cut of the key range); its waves take blocks of 64 keys in turn.  For the scores a lane owns
// one key and reads that key's row of the K page 16 bytes at a time, against the queries of all
// heads of the group (held in LDS, read as broadcasts), so K is read once for the group.  For
// the output a lane owns elements lane, lane + 64, ... of the head and walks the block's keys
// through the transposed V page, four keys per load, the probabilities again as broadcasts
// from LDS.  Running maximum, sum and accumulator per head are merged over the four waves in
// LDS, and over the cuts (when there are several) by attn_decode_merge_kernel from fp32
// partial results; the order of every sum is fixed by the shapes.
constexpr int DEC_WAVES = 4, DEC_KEYS = 64;

struct DecodeArgs {
  int H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs, splits;
  float scale;
  const float* slopes;  // as in AttnArgs
};

// GT: heads of the group handled together (a power of two, at most 8; a larger group is taken
// in chunks of 8 heads by workgroups of their own); DQ: elements of the head per lane
// (ceil(d / 64)).
template <typename T, int GT, int DQ>
__global__ __launch_bounds__(DEC_WAVES * KVF_WAVE) void attn_decode_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, T* __restrict__ out,
    float* __restrict__ part_acc, float* __restrict__ part_ml, DecodeArgs a) {
  __shared__ float Qs[GT][256];
  __shared__ float Ps[DEC_WAVES][GT][DEC_KEYS];
  __shared__ float Ms[DEC_WAVES][GT], Ls[DEC_WAVES][GT];
  __shared__ float Os[DEC_WAVES][GT][DQ * KVF_WAVE];
  const int tid = threadIdx.x, lane = tid % KVF_WAVE, wave = tid / KVF_WAVE;
  const int G = a.H / a.KV, D = a.d;
  const int chunks = (G + GT - 1) / GT;
  const int kvh = blockIdx.x / chunks, g0 = (blockIdx.x % chunks) * GT;
  const int cut = blockIdx.y, slot = blockIdx.z;
  const int seq = seq_ids ? seq_ids[slot] : slot;
  const bool seq_ok = seq >= 0 && seq < a.n_seqs;
  const int ctx = seq_ok ? ctx_lens[seq] : 0;
  const int token = seq_ok ? (cu_q ? cu_q[seq] : seq) : 0;
  const int pos = ctx - 1;
  int lo = 0;
  if (a.window > 0 && pos - a.window + 1 > 0) lo = pos - a.window + 1;
  // blocks of 64 keys from the block that holds `lo`; this cut takes blocks [b_lo, b_hi)
  const int first = lo / DEC_KEYS;
  const int n_blocks = ctx > 0 ? pos / DEC_KEYS - first + 1 : 0;
  const int per_cut = (n_blocks + a.splits - 1) / a.splits;
  const int b_lo = first + cut * per_cut, b_hi = min(first + n_blocks, b_lo + per_cut);
  const int* table = block_table + static_cast<size_t>(seq_ok ? seq : 0) * a.table_stride;

  for (int idx = tid; idx < GT * D; idx += DEC_WAVES * KVF_WAVE) {
    const int g = idx / D, kk = idx - g * D;
    Qs[g][kk] = (g0 + g < G && ctx > 0)
                    ? Elem<T>::load(q + static_cast<size_t>(token) * a.q_stride + (kvh * G + g0 + g) * D + kk)
                    : 0.f;
  }
  __syncthreads();

  float m_run[GT], l_run[GT], acc[GT][DQ], slope[GT];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    slope[g] = a.slopes && g0 + g < G ? a.slopes[kvh * G + g0 + g] : 0.f;
    m_run[g] = -INFINITY;
    l_run[g] = 0.f;
#pragma unroll
    for (int i = 0; i < DQ; ++i) acc[g][i] = 0.f;
  }
  const bool quads = a.block_size % 4 == 0;
  for (int b = b_lo + wave; b < b_hi; b += DEC_WAVES) {
    const int j = b * DEC_KEYS + lane;  // this lane's key
    const bool vis = j >= lo && j <= pos;
    // the page of every key of the context, visible or not: the values of four neighbouring keys
    // are read together further down, and a hidden one among them only has probability zero
    int page = -1;
    if (j <= pos) {
      const int blk = j / a.block_size;
      page = blk < a.table_stride ? table[blk] : -1;
      if (page >= a.num_blocks) page = -1;
    }
    const int off = j % a.block_size;
    float s[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) s[g] = 0.f;
    if (vis && page >= 0) {
      const T* krow = k_pages + ((static_cast<size_t>(page) * a.KV + kvh) * a.block_size + off) * D;
      for (int kc = 0; kc < D; kc += 16) {
        float kv[16];
        load8(krow + kc, *reinterpret_cast<float(*)[8]>(&kv[0]));
        load8(krow + kc + 8, *reinterpret_cast<float(*)[8]>(&kv[8]));
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          float t = s[g];
#pragma unroll
          for (int e = 0; e < 16; ++e) t = fmaf(Qs[g][kc + e], kv[e], t);
          s[g] = t;
        }
      }
    }
    float corr[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      const float sc = (vis && page >= 0) ? fmaf(slope[g], static_cast<float>(j - pos), s[g] * a.scale) : -INFINITY;
      const float m_new = fmaxf(m_run[g], wave_max(sc));
      float p = 0.f;
      corr[g] = 1.f;
      if (m_new > -INFINITY) {
        corr[g] = expf(m_run[g] - m_new);  // 0 on the first block with a visible key
        p = expf(sc - m_new);
      }
      Ps[wave][g][lane] = p;
      l_run[g] = l_run[g] * corr[g] + wave_sum(p);
      m_run[g] = m_new;
#pragma unroll
      for (int i = 0; i < DQ; ++i) acc[g][i] *= corr[g];
    }
    // ---- output: elements lane + 64 i over the block's keys
    const int step = quads ? 4 : 1;
    for (int c = 0; c < DEC_KEYS; c += step) {
      // keys c .. c+3 share a page when pages hold a multiple of four; no page: the keys lie
      // beyond the context or in a page that a window has given back
      const int pg = __shfl(page, c, KVF_WAVE);
      if (pg < 0) continue;
      const int o = (b * DEC_KEYS + c) % a.block_size;
#pragma unroll
      for (int i = 0; i < DQ; ++i) {
        const int e = lane + KVF_WAVE * i;
        if (e >= D) continue;
        const T* vp = v_pages + ((static_cast<size_t>(pg) * a.KV + kvh) * D + e) * a.block_size + o;
        if (quads) {
          float v4[4];
          if (sizeof(T) == 4) {
            const float4 r = *reinterpret_cast<const float4*>(vp);
            v4[0] = r.x; v4[1] = r.y; v4[2] = r.z; v4[3] = r.w;
          } else {
            const uint2 r = *reinterpret_cast<const uint2*>(vp);
            v4[0] = __uint_as_float(r.x << 16); v4[1] = __uint_as_float(r.x & 0xffff0000u);
            v4[2] = __uint_as_float(r.y << 16); v4[3] = __uint_as_float(r.y & 0xffff0000u);
          }
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            float t = acc[g][i];
#pragma unroll
            for (int x = 0; x < 4; ++x) t = fmaf(Ps[wave][g][c + x], v4[x], t);  // hidden keys have p = 0
            acc[g][i] = t;
          }
        } else {
          const float v = Elem<T>::load(vp);
#pragma unroll
          for (int g = 0; g < GT; ++g) acc[g][i] = fmaf(Ps[wave][g][c], v, acc[g][i]);
        }
      }
    }
  }
  // ---- the four waves' results into one
  if (lane < GT) {
    float mv = -INFINITY, lv = 0.f;
#pragma unroll
    for (int g = 0; g < GT; ++g)
      if (g == lane) { mv = m_run[g]; lv = l_run[g]; }
    Ms[wave][lane] = mv;
    Ls[wave][lane] = lv;
  }
#pragma unroll
  for (int g = 0; g < GT; ++g)
#pragma unroll
    for (int i = 0; i < DQ; ++i) Os[wave][g][lane + KVF_WAVE * i] = acc[g][i];
  __syncthreads();
  if (!seq_ok) return;
  for (int idx = tid; idx < min(GT, G - g0) * D; idx += DEC_WAVES * KVF_WAVE) {
    const int g = idx / D, e = idx - g * D;
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) m = fmaxf(m, Ms[w][g]);
    float l = 0.f, o = 0.f;
    if (m > -INFINITY) {
#pragma unroll
      for (int w = 0; w < DEC_WAVES; ++w) {
        const float f = expf(Ms[w][g] - m);   // exp(-inf) = 0 for a wave that saw no key
        l += Ls[w][g] * f;
        o += Os[w][g][e] * f;
      }
    }
    const int head = kvh * G + g0 + g;
    if (a.splits == 1) {
      // a sequence without context (padding of a captured batch) gets zeros, as the merge
      // kernel gives it: no row of the output keeps what an earlier step left there
      Elem<T>::store(out + static_cast<size_t>(token) * a.o_stride + head * D + e,
                     l > 0.f ? o / l : 0.f);
    } else {
      const size_t p = (static_cast<size_t>(slot) * a.H + head) * a.splits + cut;
      part_acc[p * D + e] = o;
      if (e == 0) {
        part_ml[2 * p] = m;
        part_ml[2 * p + 1] = l;
      }
    }
  }
}

// One workgroup per (sequence slot, head): the cuts' partial results into the output row, in
// cut order.  A sequence without context (padding of a captured batch) gets a row of zeros.
template <typename T>
__global__ __launch_bounds__(KVF_WAVE) void attn_decode_merge_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    const int* __restrict__ seq_ids, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    T* __restrict__ out, DecodeArgs a) {
  const int head = blockIdx.x, slot = blockIdx.y;
  const int seq = seq_ids ? seq_ids[slot] : slot;
  if (seq < 0 || seq >= a.n_seqs) return;
  const int token = cu_q ? cu_q[seq] : seq;
  if (ctx_lens[seq] <= 0) {
    for (int e = threadIdx.x; e < a.d; e += KVF_WAVE)
      Elem<T>::store(out + static_cast<size_t>(token) * a.o_stride + head * a.d + e, 0.f);
    return;
  }
  const size_t p0 = (static_cast<size_t>(slot) * a.H + head) * a.splits;
  float m = -INFINITY;
  for (int c = 0; c < a.splits; ++c) m = fmaxf(m, part_ml[2 * (p0 + c)]);
  for (int e = threadIdx.x; e < a.d; e += KVF_WAVE) {
    float l = 0.f, o = 0.f;
    if (m > -INFINITY) {
      for (int c = 0; c < a.splits; ++c) {
        const float f = expf(part_ml[2 * (p0 + c)] - m);
        l += part_ml[2 * (p0 + c) + 1] * f;
        o += part_acc[(p0 + c) * a.d + e] * f;
      }
    }
    Elem<T>::store(out + static_cast<size_t>(token) * a.o_stride + head * a.d + e, l > 0.f ? o / l : 0.f);
  }
}

template <typename T, int GT>
int launch_decode_g(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                    const int* seq_ids, const int* cu_q, const int* ctx_lens, void* out,
                    float* part_acc, float* part_ml, int num_seqs, DecodeArgs a, hipStream_t s) {
  const int G = a.H / a.KV;
  dim3 grid(a.KV * ((G + GT - 1) / GT), a.splits, num_seqs);
#define GO(DQ)                                                                                    \
  hipLaunchKernelGGL((attn_decode_kernel<T, GT, DQ>), grid, dim3(DEC_WAVES * KVF_WAVE), 0, s,     \
                     static_cast<const T*>(q), static_cast<const T*>(k_pages),                    \
                     static_cast<const T*>(v_pages), block_table, seq_ids, cu_q, ctx_lens,        \
                     static_cast<T*>(out), part_acc, part_ml, a)
  if (a.d <= 64) GO(1);
  else if (a.d <= 128) GO(2);
  else GO(4);
#undef GO
  int code = kvf_last_error();
  if (code != 0 || a.splits == 1) return code;
  hipLaunchKernelGGL((attn_decode_merge_kernel<T>), dim3(a.H, num_seqs), dim3(KVF_WAVE), 0, s, part_acc,
                     part_ml, seq_ids, cu_q, ctx_lens, static_cast<T*>(out), a);
  return kvf_last_error();
}

template <typename T>
int launch_decode(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                  const int* seq_ids, const int* cu_q, const int* ctx_lens, void* out,
                  float* part_acc, float* part_ml, int num_seqs, DecodeArgs a, hipStream_t s) {
  const int G = a.H / a.KV;
#define GO(GT)                                                                                     \
  return launch_decode_g<T, GT>(q, k_pages, v_pages, block_table, seq_ids, cu_q, ctx_lens, out,    \
                                part_acc, part_ml, num_seqs, a, s)
  if (G <= 1) GO(1);
  if (G <= 2) GO(2);
  if (G <= 4) GO(4);
  GO(8);
#undef GO
}
}  // namespace

// Single-token queries: sequence slots 0..num_seqs-1 are the sequences seq_ids[slot] (or the
// slots themselves when seq_ids is null); a sequence's token is cu_q[seq] (or seq when cu_q is
// null).  splits > 1 cuts every key range into that many runs of whole blocks of 64 keys and
// needs part_acc (num_seqs * H * splits * d floats) and part_ml (num_seqs * H * splits * 2).
KVF_EXPORT int kvf_attn_generic_decode(int dtype, const void* q, const void* k_pages,
                                       const void* v_pages, const int* block_table,
                                       const int* seq_ids, const int* cu_q, const int* ctx_lens,
                                       void* out, float* part_acc, float* part_ml, int num_seqs,
                                       int H, int KV, int d, int block_size, int num_blocks,
                                       int table_stride, int q_stride, int o_stride, int window,
                                       int n_seqs, int splits, float scale, const float* slopes,
                                       hipStream_t s) {
  if (num_seqs <= 0) return 0;
  if (d % 16 != 0 || d > 256 || d <= 0 || KV <= 0 || H % KV != 0 || splits < 1 ||
      (splits > 1 && (!part_acc || !part_ml)) || block_size <= 0)
    return static_cast<int>(hipErrorInvalidValue);
  DecodeArgs a{H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs,
               splits, scale, slopes};
  if (dtype == 0)
    return launch_decode<float>(q, k_pages, v_pages, block_table, seq_ids, cu_q, ctx_lens, out,
                                part_acc, part_ml, num_seqs, a, s);
  if (dtype == 1)
    return launch_decode<bf16_t>(q, k_pages, v_pages, block_table, seq_ids, cu_q, ctx_lens, out,
                                 part_acc, part_ml, num_seqs, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}

// dtype: 0 = fp32, 1 = bf16.  d must be a multiple of 16 and at most 256 (checked by the caller
// and here).  `work` holds num_work rows (sequence, item, item or -1), an item being
// kvf_attn_generic_rows_per_item() rows of (query token, head in the kv head's group).
KVF_EXPORT int kvf_attn_generic(int dtype, const void* q, const void* k_pages, const void* v_pages,
                                const int* block_table, const int* cu_q, const int* ctx_lens,
                                const int* work, int num_work, void* out, int H, int KV, int d,
                                int block_size, int num_blocks, int table_stride, int q_stride,
                                int o_stride, int window, int n_seqs, float scale,
                                const float* slopes, hipStream_t s) {
  if (d % 16 != 0 || d > 256 || d <= 0 || KV <= 0 || H % KV != 0 || !work || block_size <= 0 ||
      q_stride % 4 != 0 || o_stride % 4 != 0)
    return static_cast<int>(hipErrorInvalidValue);
  AttnArgs a{H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs,
             scale, slopes};
  if (dtype == 0)
    return launch<float>(q, k_pages, v_pages, block_table, cu_q, ctx_lens, work, num_work, out, a, s);
  if (dtype == 1)
    return launch<bf16_t>(q, k_pages, v_pages, block_table, cu_q, ctx_lens, work, num_work, out, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}

KVF_EXPORT int kvf_attn_generic_rows_per_item() { return ITEM_ROWS; }
