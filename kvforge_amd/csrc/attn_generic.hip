// Paged causal attention for query runs of any length, computed on the vector ALUs in fp32.
// It is the attention of the true 32-bit path and takes bf16 operands as well.
//
// One workgroup handles 16 "rows" of one (sequence, kv head): row r of a sequence is
// (query token r / G, head r % G of the kv head's group), so the G query heads that share a
// kv head also share every K/V tile the workgroup loads.  Keys are walked in tiles aligned
// to multiples of the tile size from position 0, with a running maximum, sum and accumulator
// per row (all fp32).  Key j is visible to the query at position p iff j <= p, j < context
// length and, with a window w > 0, j > p - w.  Scores are scaled after the dot product.
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
      s[jj] = vis ? s[jj] * a.scale : -INFINITY;
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
}  // namespace

// dtype: 0 = fp32, 1 = bf16.  d must be a multiple of 16 and at most 256 (checked by the caller
// and here).  tiles_per_seq == 0: `work` holds num_work rows (sequence, 16-row tile, tile or -1).
// tiles_per_seq > 0: num_work sequences, listed in `work` or 0..num_work-1 when it is null, each
// with that many tiles (single-token queries need ceil(G / 16)).
KVF_EXPORT int kvf_attn_generic(int dtype, const void* q, const void* k_pages, const void* v_pages,
                                const int* block_table, const int* cu_q, const int* ctx_lens,
                                const int* work, int num_work, int tiles_per_seq, void* out, int H,
                                int KV, int d, int block_size, int num_blocks, int table_stride,
                                int q_stride, int o_stride, int window, int n_seqs, float scale,
                                hipStream_t s) {
  if (d % 16 != 0 || d > 256 || d <= 0 || KV <= 0 || H % KV != 0 || tiles_per_seq < 0 ||
      (tiles_per_seq == 0 && !work))
    return static_cast<int>(hipErrorInvalidValue);
  AttnArgs a{H, KV, d, block_size, num_blocks, table_stride, q_stride, o_stride, window, n_seqs,
             tiles_per_seq, scale};
  num_work *= tiles_per_seq > 0 ? tiles_per_seq : 2;
  if (dtype == 0)
    return launch<float>(q, k_pages, v_pages, block_table, cu_q, ctx_lens, work, num_work, out, a, s);
  if (dtype == 1)
    return launch<bf16_t>(q, k_pages, v_pages, block_table, cu_q, ctx_lens, work, num_work, out, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}
