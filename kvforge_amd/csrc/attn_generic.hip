// Paged causal attention for query runs of any length, computed on the vector ALUs in fp32.
// It is the attention of the true 32-bit path and takes bf16 operands as well.
//
// One workgroup handles 16 "rows" of one (sequence, kv head): row r of a sequence is
// (query token r / G, head r % G of the kv head's group), so the G query heads that share a
// kv head also share every K/V tile the workgroup loads.  Keys are walked in tiles aligned
// to multiples of the tile size from position 0, with a running maximum, sum and accumulator
// per row (all fp32).  Key j is visible to the query at position p iff j <= p, j < context
// length and, with a window w > 0, j > p - w.  Scores are scaled after the dot product; with
// `slopes` (one number per q head) slopes[h] * (j - p) is added to them, a bias by distance.
//
// K pages are [num_blocks, KV, block_size, d], V pages are transposed [num_blocks, KV, d,
// block_size]; a key whose page entry is negative or out of range contributes nothing.
#include "common.h"

namespace {
constexpr int ROWS = 16;

struct AttnArgs {
  int H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs;
  int tiles_per_seq;  // 0: `work` holds (sequence, tile, tile or -1) rows; > 0: `work` lists sequences (or
                      // is null for 0, 1, 2, ...) and each takes this many tiles
  float scale;
  const float* slopes;  // null, or one number per q head: slopes[h] * (key - query position) is added to a score
};

template <typename T, int DMAX, int BKEYS>
__global__ __launch_bounds__(256) void attn_tile_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens, const int* __restrict__ work, T* __restrict__ out,
    AttnArgs a) {
  __shared__ float Qs[ROWS][DMAX + 1];
  __shared__ float KVs[BKEYS][DMAX + 1];
  __shared__ float Ps[ROWS][BKEYS + 1];

  int seq, tile;
  if (a.tiles_per_seq > 0) {
    const int idx = blockIdx.x / a.tiles_per_seq;
    seq = work ? work[idx] : idx;
    tile = blockIdx.x - idx * a.tiles_per_seq;
  } else {
    // rows (sequence, tile, tile or -1): two workgroups per row, one for each tile
    const int w = blockIdx.x >> 1;
    seq = work[3 * w];
    tile = work[3 * w + 1 + (blockIdx.x & 1)];
    if (tile < 0) return;
  }
  if (seq < 0 || seq >= a.n_seqs) return;
  const int kvh = blockIdx.y;
  const int G = a.H / a.KV, D = a.d;
  const int q0 = cu_q[seq], qlen = cu_q[seq + 1] - q0, ctx = ctx_lens[seq];
  const int start = ctx - qlen;  // position of the run's first query
  const int rows_total = qlen * G, r0 = tile * ROWS;
  if (r0 >= rows_total || qlen <= 0 || start < 0) return;

  const int tid = threadIdx.x;
  const int r = tid / 16, c16 = tid % 16;
  const int* table = block_table + static_cast<size_t>(seq) * a.table_stride;

  // stage the query rows
  for (int idx = tid; idx < ROWS * D; idx += 256) {
    const int rr = idx / D, kk = idx - rr * D;
    const int row = r0 + rr;
    float v = 0.f;
    if (row < rows_total) {
      const int i = row / G, g = row - i * G;
      v = Elem<T>::load(q + static_cast<size_t>(q0 + i) * a.q_stride + (kvh * G + g) * D + kk);
    }
    Qs[rr][kk] = v;
  }

  const int my_row = r0 + r;
  const bool row_ok = my_row < rows_total;
  const int my_pos = start + (row_ok ? my_row / G : 0);
  const float slope = a.slopes && row_ok ? a.slopes[kvh * G + my_row % G] : 0.f;
  const int pos_min = start + r0 / G;
  int last_row = r0 + ROWS - 1;
  if (last_row >= rows_total) last_row = rows_total - 1;
  const int pos_max = start + last_row / G;
  int lo = 0;
  if (a.window > 0) {
    lo = pos_min - a.window + 1;
    if (lo < 0) lo = 0;
  }
  const int hi = pos_max < ctx - 1 ? pos_max : ctx - 1;  // last key any row may see

  float m_run = -INFINITY, l_run = 0.f;
  float acc[DMAX / 16];
#pragma unroll
  for (int j = 0; j < DMAX / 16; ++j) acc[j] = 0.f;

  const int chunks_per_key = D / 8;
  for (int t0 = (lo / BKEYS) * BKEYS; t0 <= hi; t0 += BKEYS) {
    // ---- K tile
    __syncthreads();
    for (int ch = tid; ch < BKEYS * chunks_per_key; ch += 256) {
      const int c = ch / chunks_per_key, k8 = (ch - c * chunks_per_key) * 8;
      const int j = t0 + c;
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (j >= lo && j <= hi) {
        const int blk = j / a.block_size;
        const int page = blk < a.table_stride ? table[blk] : -1;
        if (page >= 0 && page < a.num_blocks)
          load8(k_pages + ((static_cast<size_t>(page) * a.KV + kvh) * a.block_size +
                           (j - blk * a.block_size)) * D + k8, v);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) KVs[c][k8 + e] = v[e];
    }
    __syncthreads();
    // ---- scores for row r, keys c16 + 16*jj
    float s[BKEYS / 16];
#pragma unroll
    for (int jj = 0; jj < BKEYS / 16; ++jj) s[jj] = 0.f;
    for (int kk = 0; kk < D; ++kk) {
      const float qv = Qs[r][kk];
#pragma unroll
      for (int jj = 0; jj < BKEYS / 16; ++jj) s[jj] = fmaf(qv, KVs[c16 + 16 * jj][kk], s[jj]);
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int jj = 0; jj < BKEYS / 16; ++jj) {
      const int j = t0 + c16 + 16 * jj;
      bool vis = row_ok && j <= my_pos && j < ctx;
      if (a.window > 0) vis = vis && (j > my_pos - a.window);
      s[jj] = vis ? fmaf(slope, static_cast<float>(j - my_pos), s[jj] * a.scale) : -INFINITY;
      tmax = fmaxf(tmax, s[jj]);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, KVF_WAVE));
    const float m_new = fmaxf(m_run, tmax);
    float corr = 1.f, psum = 0.f;
    if (m_new == -INFINITY) {
#pragma unroll
      for (int jj = 0; jj < BKEYS / 16; ++jj) Ps[r][c16 + 16 * jj] = 0.f;
    } else {
      corr = expf(m_run - m_new);  // exp(-inf) = 0 on the first visible tile
#pragma unroll
      for (int jj = 0; jj < BKEYS / 16; ++jj) {
        const float p = expf(s[jj] - m_new);
        Ps[r][c16 + 16 * jj] = p;
        psum += p;
      }
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, KVF_WAVE);
    l_run = l_run * corr + psum;
    m_run = m_new;
#pragma unroll
    for (int j = 0; j < DMAX / 16; ++j) acc[j] *= corr;
    // ---- V tile (overwrites the K tile once every thread has finished with it); V pages hold
    // the keys of one element side by side, so a thread walks keys fastest
    __syncthreads();
    for (int idx = tid; idx < BKEYS * D; idx += 256) {
      const int e = idx / BKEYS, c = idx - e * BKEYS;
      const int j = t0 + c;
      float v = 0.f;
      if (j >= lo && j <= hi) {
        const int blk = j / a.block_size;
        const int page = blk < a.table_stride ? table[blk] : -1;
        if (page >= 0 && page < a.num_blocks)
          v = Elem<T>::load(v_pages + ((static_cast<size_t>(page) * a.KV + kvh) * D + e) * a.block_size +
                            (j - blk * a.block_size));
      }
      KVs[c][e] = v;
    }
    __syncthreads();
    for (int c = 0; c < BKEYS; ++c) {
      const float p = Ps[r][c];
#pragma unroll
      for (int j = 0; j < DMAX / 16; ++j)
        if (c16 + 16 * j < D) acc[j] = fmaf(p, KVs[c][c16 + 16 * j], acc[j]);
    }
  }
  if (!row_ok) return;
  const int i = my_row / G, g = my_row - i * G;
  T* o = out + static_cast<size_t>(q0 + i) * a.o_stride + (kvh * G + g) * D;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
  for (int j = 0; j < DMAX / 16; ++j)
    if (c16 + 16 * j < D) Elem<T>::store(o + c16 + 16 * j, acc[j] * inv);
}

template <typename T>
int launch(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
           const int* cu_q, const int* ctx_lens, const int* work, int num_work, void* out,
           AttnArgs a, hipStream_t s) {
  if (num_work <= 0) return 0;
  dim3 grid(num_work, a.KV);
#define GO(DMAX, BKEYS)                                                                           \
  hipLaunchKernelGGL((attn_tile_kernel<T, DMAX, BKEYS>), grid, dim3(256), 0, s,                   \
                     static_cast<const T*>(q), static_cast<const T*>(k_pages),                    \
                     static_cast<const T*>(v_pages), block_table, cu_q, ctx_lens, work,           \
                     static_cast<T*>(out), a)
  if (a.d <= 64) GO(64, 64);
  else if (a.d <= 128) GO(128, 64);
  else GO(256, 32);
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
// and here).  tiles_per_seq == 0: `work` holds num_work rows (sequence, 16-row tile, tile or -1).
// tiles_per_seq > 0: num_work sequences, listed in `work` or 0..num_work-1 when it is null, each
// with that many tiles (single-token queries need ceil(G / 16)).
KVF_EXPORT int kvf_attn_generic(int dtype, const void* q, const void* k_pages, const void* v_pages,
                                const int* block_table, const int* cu_q, const int* ctx_lens,
                                const int* work, int num_work, int tiles_per_seq, void* out, int H,
                                int KV, int d, int block_size, int num_blocks, int table_stride,
                                int q_stride, int o_stride, int window, int n_seqs, float scale,
                                const float* slopes, hipStream_t s) {
  if (d % 16 != 0 || d > 256 || d <= 0 || KV <= 0 || H % KV != 0 || tiles_per_seq < 0 ||
      (tiles_per_seq == 0 && !work))
    return static_cast<int>(hipErrorInvalidValue);
  AttnArgs a{H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs,
             tiles_per_seq, scale, slopes};
  num_work *= tiles_per_seq > 0 ? tiles_per_seq : 2;
  if (dtype == 0)
    return launch<float>(q, k_pages, v_pages, block_table, cu_q, ctx_lens, work, num_work, out, a, s);
  if (dtype == 1)
    return launch<bf16_t>(q, k_pages, v_pages, block_table, cu_q, ctx_lens, work, num_work, out, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}
