// Paged causal attention for bf16 on the matrix cores, for query runs (prefill) and for single
// tokens (decode).  No tile of K or V passes through LDS: every operand fragment is loaded
// from the pages straight into the registers layout the instruction wants.
//
// Rows: row r of a (sequence, kv head) is (query token r / G, head r % G of the group), so the
// G query heads that share a kv head share every K/V fragment.  A wave owns tiles of 16 rows;
// lane l belongs to row l % 16 for the whole kernel, so the running maximum, sum and rescale
// factor of a row are plain per-lane scalars (fp32).
//
// Keys are walked in blocks of 32.  For a block starting at kb, with lane group g = l / 16:
//   S^T (keys x rows) = K (keys x d) * Q^T: two v_mfma_f32_16x16x32_bf16 tiles t = 0, 1 whose
//   16 key rows are chosen as  kb + 8*(i/4) + 4*t + i%4,  i = 0..15.  Lane group g then holds the
//   scores of keys kb + 8g + 4t + {0..3}: over both tiles the eight neighbouring keys
//   kb + 8g .. kb + 8g + 7 - exactly the contraction slots a lane feeds to the second product.
//   O^T (d x rows) += V^T (d x keys) * P^T (keys x rows): V pages are stored transposed,
//   [num_blocks, KV, d, block_size], so a lane's eight keys of one element are 16 contiguous
//   bytes.  Probabilities go from the first product's accumulators to the second product's
//   operand by a rounding to bf16 alone; softmax itself is fp32.
// Key j is visible to a query at position p iff j <= p, j < context length and, with a window
// w > 0, j > p - w.  Scores are scaled after the dot product.
//
// SPLIT = false (runs): a workgroup takes 4 * RT consecutive row tiles of one (sequence, kv
//   head) from a work list; its waves are independent.
// SPLIT = true (few rows, long key range): a workgroup takes one row tile and one of `splits`
//   cuts of the key range; its four waves take the blocks of that cut in turn and are merged
//   through LDS; with splits > 1 partial (max, sum, accumulator) go to a workspace that
//   `attn_split_combine_kernel` merges in split order.
// block_size must be a multiple of 8 (a lane's eight keys lie in one page), d a multiple of 16.
#include "common.h"

namespace {
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
constexpr int WAVES = 4;

struct MArgs {
  int H, KV, d, bs, nb, table_stride, q_stride, o_stride, window, n_seqs, splits;
  float scale;
};

__device__ __forceinline__ bf16x8 ld_frag(const bf16_t* p, bool ok) {
  uint4 r = make_uint4(0u, 0u, 0u, 0u);
  if (ok) r = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, r);
}

// max over the four lanes of a row (lanes j, j+16, j+32, j+48)
__device__ __forceinline__ float row_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, KVF_WAVE));
  return fmaxf(v, __shfl_xor(v, 32, KVF_WAVE));
}
__device__ __forceinline__ float row_sum(float v) {
  v += __shfl_xor(v, 16, KVF_WAVE);
  return v + __shfl_xor(v, 32, KVF_WAVE);
}

template <int DTMAX, int RT, bool SPLIT>
__global__ __launch_bounds__(256) void attn_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ vt_pages, const int* __restrict__ block_table,
    const int* __restrict__ items, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    bf16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml, MArgs a) {
  constexpr int DCMAX = DTMAX / 2;  // 32-wide steps of the q.k contraction
  extern __shared__ float lds[];    // SPLIT only: [WAVES][dt][64][4] accumulators, [WAVES][16][2]

  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int j16 = lane % 16, kg = lane / 16;
  const int G = a.H / a.KV, D = a.d;
  const int dt_n = D / 16, dc_n = (D + 31) / 32;

  int seq, kvh, first_tile, item_index;
  if (SPLIT) {
    const int chunks = (G + 15) / 16;
    item_index = blockIdx.x;
    seq = items ? items[blockIdx.x] : static_cast<int>(blockIdx.x);
    kvh = blockIdx.y / chunks;
    first_tile = blockIdx.y - kvh * chunks;
  } else {
    item_index = 0;
    seq = items[2 * blockIdx.x];
    kvh = blockIdx.y;
    first_tile = (items[2 * blockIdx.x + 1] * WAVES + wave) * RT;
  }
  if (seq < 0 || seq >= a.n_seqs) return;
  const int q0 = cu_q[seq], qlen = cu_q[seq + 1] - q0, ctx = ctx_lens[seq];
  const int start = ctx - qlen;
  const int rows_total = qlen * G;
  const int* table = block_table + static_cast<size_t>(seq) * a.table_stride;
  const bool seq_ok = qlen > 0 && start >= 0;

  // ---- this lane's rows and their query fragments
  bool row_ok[RT];
  int row_pos[RT], row_tok[RT], row_head[RT];
  bf16x8 qf[RT][DCMAX];
  int pos_min = 0x7fffffff, pos_max = -1;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = (first_tile + rt) * 16 + j16;
    row_ok[rt] = seq_ok && row < rows_total;
    const int tok = row_ok[rt] ? row / G : 0;
    row_tok[rt] = tok;
    row_head[rt] = kvh * G + (row_ok[rt] ? row - tok * G : 0);
    row_pos[rt] = start + tok;
    const int t_lo = (first_tile + rt) * 16 / G;                       // first token of the tile
    int t_hi = ((first_tile + rt) * 16 + 15) / G;                      // last token of the tile
    if (t_hi > qlen - 1) t_hi = qlen - 1;
    if (seq_ok && (first_tile + rt) * 16 < rows_total) {
      pos_min = min(pos_min, start + t_lo);
      pos_max = max(pos_max, start + t_hi);
    }
    const bf16_t* qp = q + static_cast<size_t>(q0 + tok) * a.q_stride + row_head[rt] * D + kg * 8;
#pragma unroll
    for (int c = 0; c < DCMAX; ++c)
      qf[rt][c] = ld_frag(qp + c * 32, row_ok[rt] && c < dc_n && c * 32 + kg * 8 < D);
  }
  // ---- key range of this wave
  int lo = 0, hi = -1;
  if (pos_max >= 0) {
    hi = pos_max < ctx - 1 ? pos_max : ctx - 1;
    if (a.window > 0 && pos_min - a.window + 1 > 0) lo = pos_min - a.window + 1;
  }
  int kb_begin = (lo / 32) * 32, kb_step = 32, kb_end = hi + 1;
  if (SPLIT) {
    const int blocks = hi >= kb_begin ? (hi - kb_begin) / 32 + 1 : 0;
    int per = (blocks + a.splits - 1) / a.splits;
    per = (per + WAVES - 1) / WAVES * WAVES;          // whole rounds of the four waves
    const int b0 = blockIdx.z * per;
    kb_end = min(kb_end, kb_begin + (b0 + per) * 32);
    kb_begin += (b0 + wave) * 32;
    kb_step = 32 * WAVES;
  }

  float m_run[RT], l_run[RT];
  f32x4 acc[RT][DTMAX];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m_run[rt] = -INFINITY;
    l_run[rt] = 0.f;
#pragma unroll
    for (int t = 0; t < DTMAX; ++t) acc[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  for (int kb = kb_begin; kb < kb_end; kb += kb_step) {
    // ---- K fragments: tile t, row i = j16 is key kb + 8*(i/4) + 4*t + i%4
    bf16x8 kf[2][DCMAX];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = kb + 8 * (j16 >> 2) + 4 * t + (j16 & 3);
      const int blk = key / a.bs;
      int page = -1;
      if (key < ctx && blk < a.table_stride) page = table[blk];
      const bool ok = page >= 0 && page < a.nb;
      const bf16_t* kp = k_pages + ((static_cast<size_t>(ok ? page : 0) * a.KV + kvh) * a.bs +
                                    (key - blk * a.bs)) * D + kg * 8;
#pragma unroll
      for (int c = 0; c < DCMAX; ++c)
        kf[t][c] = ld_frag(kp + c * 32, ok && c < dc_n && c * 32 + kg * 8 < D);
    }
    // ---- V^T fragments: row i = j16 is element dt*16 + i, slots are keys kb + 8*kg + 0..7
    bf16x8 vf[DTMAX];
    {
      const int key = kb + 8 * kg;
      const int blk = key / a.bs;
      int page = -1;
      if (key < ctx && blk < a.table_stride) page = table[blk];
      const bool ok = page >= 0 && page < a.nb;
      const bf16_t* vp = vt_pages + ((static_cast<size_t>(ok ? page : 0) * a.KV + kvh) * D + j16) * a.bs +
                         (key - blk * a.bs);
      // keys at or past the context length hold whatever an earlier owner left: clear them
      const int live = ctx - key;  // > 0 when ok
#pragma unroll
      for (int t = 0; t < DTMAX; ++t) {
        vf[t] = ld_frag(vp + static_cast<size_t>(t) * 16 * a.bs, ok && t < dt_n);
        if (ok && live < 8) {
          uint4 r = __builtin_bit_cast(uint4, vf[t]);
          uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (2 * e >= live) w[e] = 0u;
            else if (2 * e + 1 >= live) w[e] &= 0xffffu;
          }
          vf[t] = __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
        }
      }
    }
    const bool edge = kb + 31 > pos_min || kb + 32 > ctx || a.window > 0;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      f32x4 s[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DCMAX; ++c)
          if (c < dc_n) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][c], qf[rt][c], s[t], 0, 0, 0);
      }
      // lane holds keys kb + 8*kg + 4*t + r of row j16
      float bm = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = s[t][r] * a.scale;
          if (edge) {
            const int key = kb + 8 * kg + 4 * t + r;
            bool vis = row_ok[rt] && key <= row_pos[rt] && key < ctx;
            if (a.window > 0) vis = vis && key > row_pos[rt] - a.window;
            if (!vis) v = -INFINITY;
          } else if (!row_ok[rt]) {
            v = -INFINITY;
          }
          s[t][r] = v;
          bm = fmaxf(bm, v);
        }
      bm = row_max(bm);
      const float m_new = fmaxf(m_run[rt], bm);
      float p[8], corr = 1.f, psum = 0.f;
      if (m_new == -INFINITY) {
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = 0.f;
      } else {
        corr = __expf(m_run[rt] - m_new);  // exp(-inf) = 0 on the first visible block
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            p[4 * t + r] = __expf(s[t][r] - m_new);
            psum += p[4 * t + r];
          }
      }
      l_run[rt] = l_run[rt] * corr + psum;  // this lane's share of the row's sum
      m_run[rt] = m_new;
      typedef __attribute__((ext_vector_type(8))) float f32x8;
      f32x8 pv;
#pragma unroll
      for (int e = 0; e < 8; ++e) pv[e] = p[e];
      const bf16x8 pf = __builtin_convertvector(pv, bf16x8);
#pragma unroll
      for (int t = 0; t < DTMAX; ++t)
        if (t < dt_n) {
          acc[rt][t] *= corr;
          acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t], pf, acc[rt][t], 0, 0, 0);
        }
    }
  }

  if (!SPLIT) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const float l = row_sum(l_run[rt]);
      if (!row_ok[rt]) continue;
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16_t* o = out + static_cast<size_t>(q0 + row_tok[rt]) * a.o_stride + row_head[rt] * D + 4 * kg;
#pragma unroll
      for (int t = 0; t < DTMAX; ++t)
        if (t < dt_n) {
          uint2 pk;
          pk.x = static_cast<uint32_t>(f32_to_bf16(acc[rt][t][0] * inv)) |
                 (static_cast<uint32_t>(f32_to_bf16(acc[rt][t][1] * inv)) << 16);
          pk.y = static_cast<uint32_t>(f32_to_bf16(acc[rt][t][2] * inv)) |
                 (static_cast<uint32_t>(f32_to_bf16(acc[rt][t][3] * inv)) << 16);
          *reinterpret_cast<uint2*>(o + t * 16) = pk;
        }
    }
    return;
  }

  // ---- SPLIT: merge the four waves (RT == 1), then store or hand on the partial result
  float* red_acc = lds;                                   // [WAVES][dt_n][64][4]
  float* red_ml = lds + WAVES * dt_n * KVF_WAVE * 4;      // [WAVES][16][2]
  const float l_row = row_sum(l_run[0]);
#pragma unroll
  for (int t = 0; t < DTMAX; ++t)
    if (t < dt_n)
      *reinterpret_cast<f32x4*>(red_acc + ((wave * dt_n + t) * KVF_WAVE + lane) * 4) = acc[0][t];
  if (kg == 0) {
    red_ml[(wave * 16 + j16) * 2] = m_run[0];
    red_ml[(wave * 16 + j16) * 2 + 1] = l_row;
  }
  __syncthreads();
  float mm = -INFINITY;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, red_ml[(w * 16 + j16) * 2]);
  float cw[WAVES], ll = 0.f;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const float mw = red_ml[(w * 16 + j16) * 2];
    cw[w] = mw == -INFINITY ? 0.f : __expf(mw - mm);
    ll += red_ml[(w * 16 + j16) * 2 + 1] * cw[w];
  }
  if (!row_ok[0]) return;
  const int head = row_head[0];
  const size_t slot = (static_cast<size_t>(item_index) * a.H + head) * a.splits + blockIdx.z;
  if (a.splits > 1 && wave == 0 && kg == 0) {
    part_ml[slot * 2] = mm;
    part_ml[slot * 2 + 1] = ll;
  }
  const float inv = ll > 0.f ? 1.f / ll : 0.f;
  for (int t = wave; t < dt_n; t += WAVES) {  // wave w finishes element tiles w, w + 4, ...
    f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
      o += *reinterpret_cast<const f32x4*>(red_acc + ((w * dt_n + t) * KVF_WAVE + lane) * 4) * cw[w];
    const int e0 = t * 16 + 4 * kg;
    if (a.splits == 1) {
      uint2 pk;
      pk.x = static_cast<uint32_t>(f32_to_bf16(o[0] * inv)) | (static_cast<uint32_t>(f32_to_bf16(o[1] * inv)) << 16);
      pk.y = static_cast<uint32_t>(f32_to_bf16(o[2] * inv)) | (static_cast<uint32_t>(f32_to_bf16(o[3] * inv)) << 16);
      *reinterpret_cast<uint2*>(out + static_cast<size_t>(q0 + row_tok[0]) * a.o_stride + head * D + e0) = pk;
    } else {
      *reinterpret_cast<f32x4*>(part_acc + slot * D + e0) = o;
    }
  }
}

// Merges the splits of every (sequence, head) in split order.  One query token per sequence.
__global__ void attn_split_combine_kernel(const float* __restrict__ part_acc,
                                          const float* __restrict__ part_ml,
                                          const int* __restrict__ seq_ids,
                                          const int* __restrict__ cu_q, bf16_t* __restrict__ out,
                                          int H, int D, int splits, int o_stride, int n_seqs) {
  const int seq = seq_ids ? seq_ids[blockIdx.x] : static_cast<int>(blockIdx.x);
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
      const float c = ms == -INFINITY ? 0.f : __expf(ms - mm);
      ll += part_ml[(slot0 + s) * 2 + 1] * c;
      v += part_acc[(slot0 + s) * D + e] * c;
    }
    out[static_cast<size_t>(tok) * o_stride + head * D + e].bits = f32_to_bf16(ll > 0.f ? v / ll : 0.f);
  }
}

bool args_ok(int H, int KV, int d, int bs) {
  return d > 0 && d % 16 == 0 && d <= 256 && KV > 0 && H % KV == 0 && bs > 0 && bs % 8 == 0;
}
}  // namespace

// Rows of a query run one workgroup takes: 4 waves x RT tiles x 16 rows.
KVF_EXPORT int kvf_attn_mfma_rows_per_item(int d) { return d <= 128 ? 128 : 64; }

// Query runs: `work` holds num_work pairs (sequence, item) where item i covers rows
// [i * rows_per_item, (i + 1) * rows_per_item) of the sequence's qlen * H/KV rows per kv head.
KVF_EXPORT int kvf_attn_mfma_prefill(const void* q, const void* k_pages, const void* vt_pages,
                                     const int* block_table, const int* cu_q, const int* ctx_lens,
                                     const int* work, int num_work, void* out, int H, int KV, int d,
                                     int bs, int nb, int table_stride, int q_stride, int o_stride,
                                     int window, int n_seqs, float scale, hipStream_t s) {
  if (num_work <= 0) return 0;
  if (!args_ok(H, KV, d, bs) || q_stride % 8 != 0 || o_stride % 4 != 0)
    return static_cast<int>(hipErrorInvalidValue);
  const MArgs a{H, KV, d, bs, nb, table_stride, q_stride, o_stride, window, n_seqs, 1, scale};
  const dim3 grid(num_work, KV);
#define GO(DTMAX, RT)                                                                              \
  hipLaunchKernelGGL((attn_mfma_kernel<DTMAX, RT, false>), grid, dim3(256), 0, s,                  \
                     static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),           \
                     static_cast<const bf16_t*>(vt_pages), block_table, work, cu_q, ctx_lens,      \
                     static_cast<bf16_t*>(out), nullptr, nullptr, a)
  if (d <= 64) GO(4, 2);
  else if (d <= 128) GO(8, 2);
  else GO(16, 1);
#undef GO
  return kvf_last_error();
}

// Single-token queries: sequences seq_ids[0..num_seqs) (or 0..num_seqs-1), key range cut into
// `splits`.  With splits > 1, part_acc holds num_seqs*H*splits*d floats and part_ml
// num_seqs*H*splits*2; calls that share them must not overlap.
KVF_EXPORT int kvf_attn_mfma_decode(const void* q, const void* k_pages, const void* vt_pages,
                                    const int* block_table, const int* seq_ids, const int* cu_q,
                                    const int* ctx_lens, void* out, float* part_acc, float* part_ml,
                                    int num_seqs, int H, int KV, int d, int bs, int nb,
                                    int table_stride, int q_stride, int o_stride, int window,
                                    int n_seqs, int splits, float scale, hipStream_t s) {
  if (num_seqs <= 0) return 0;
  if (!args_ok(H, KV, d, bs) || q_stride % 8 != 0 || o_stride % 4 != 0 || splits < 1 ||
      (splits > 1 && (!part_acc || !part_ml)))
    return static_cast<int>(hipErrorInvalidValue);
  const MArgs a{H, KV, d, bs, nb, table_stride, q_stride, o_stride, window, n_seqs, splits, scale};
  const int G = H / KV, chunks = (G + 15) / 16, dt = d / 16;
  const dim3 grid(num_seqs, KV * chunks, splits);
  const size_t lds = (static_cast<size_t>(WAVES) * dt * KVF_WAVE * 4 + WAVES * 16 * 2) * sizeof(float);
#define GO(DTMAX)                                                                                  \
  hipLaunchKernelGGL((attn_mfma_kernel<DTMAX, 1, true>), grid, dim3(256), lds, s,                  \
                     static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),           \
                     static_cast<const bf16_t*>(vt_pages), block_table, seq_ids, cu_q, ctx_lens,   \
                     static_cast<bf16_t*>(out), part_acc, part_ml, a)
  if (d <= 64) GO(4);
  else if (d <= 128) GO(8);
  else GO(16);
#undef GO
  int err = kvf_last_error();
  if (err || splits == 1) return err;
  hipLaunchKernelGGL(attn_split_combine_kernel, dim3(num_seqs, H), dim3(64), 0, s, part_acc,
                     part_ml, seq_ids, cu_q, static_cast<bf16_t*>(out), H, d, splits, o_stride,
                     n_seqs);
  return kvf_last_error();
}
