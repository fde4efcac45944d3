// Paged causal attention for bf16 on the matrix cores, for query runs (prefill) and for single
// tokens (decode).  Every operand fragment is loaded from the pages in the register layout the
// instruction wants (no transposes); for query runs the four waves of a workgroup share the
// fragments of a key block through LDS, each loading a quarter of them one block ahead.
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
// With `slopes` (one number per q head) a score also gets slopes[h] * (j - p), a bias by distance;
// the kernels are instantiated with and without it, so that attention without it pays nothing.
// The softmax reference of a row (what is subtracted before exp) is raised only when some score
// of the wave exceeds it by more than LAZY (in log2 units): exp(s - ref) then stays below
// 2^LAZY, sums and accumulators need no rescaling in most blocks, and the result is the same
// softmax (any reference cancels in the final division).
//
// Loads are never predicated: a lane without a valid page reads page 0 and its fragment is
// cleared by a mask when it is consumed, so nothing waits on a load before its data is needed.
//
// Query runs: an item is 4 * RT consecutive row tiles of one (sequence, kv head), one tile set per
//   wave; a workgroup takes the one or two items of a work row in turn (two: an early item with
//   a late one, so that under the causal mask every workgroup walks about as many keys; one, the
//   longest walks first in the grid, keeps more workgroups in flight and is what the engine's
//   planner hands out).  The kv head is the grid's fastest index where the grid allows it:
//   consecutive workgroups go to consecutive XCDs, so with eight kv heads an XCD walks the keys
//   of one head only and finds them in its own L2.  Three or four stages are in
//   flight: page lookups two or three blocks ahead, fragment loads one or two blocks ahead
//   (registers, then the other half of a double LDS buffer), products of this block.
// Few rows, long key range: a workgroup takes one row tile and one of `splits` cuts of the key
//   range; blocks of 32 keys go round the waves (eight, or four where the grid fills the chip) of
//   all cuts in turn, so a wave's first block does not depend on the context length and its page
//   lookups leave with the first loads.  The waves are merged through LDS; with splits > 1
//   partial (max, sum, accumulator) go to a workspace that `attn_split_combine_kernel` merges in
//   split order.
// block_size must be a multiple of 8 (a lane's eight keys lie in one page), d a multiple of 16;
// kernels are instantiated for each d / 16 so that no loop bound is left to run time.
#include "common.h"

namespace {
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
constexpr int WAVES = 4;
constexpr float LAZY = 8.f;                    // log2 headroom before a row's reference is raised
constexpr float LOG2E = 1.4426950408889634f;

// With at least two waves per SIMD asked for, a wave has at most 256 registers and the compiler
// keeps accumulators in ordinary vector registers, where the softmax rescale can reach them
// without copies from and to the accumulation registers in every block.
#define KVF_VGPR_FORM(FITS) __attribute__((amdgpu_waves_per_eu((FITS) ? 2 : 1)))

struct MArgs {
  int H, KV, d, bs, nb, table_stride, q_stride, o_stride, window, n_seqs, splits;
  int kv_fastest;  // query runs: the kv head is the grid's fastest index (see kvf_attn_mfma_prefill)
  float scale;
  unsigned bs_magic;  // floor(2^32 / bs) + 1: key / bs == mulhi(key, bs_magic) while key * bs < 2^32
  const float* slopes;  // null, or one number per q head: slopes[h] * (key - query position) is added to a score
};

// Position of a key in its page table: (page table entry, slot in the page)
__device__ __forceinline__ int block_of(const MArgs& a, int key) {
  return static_cast<int>(__umulhi(static_cast<unsigned>(key), a.bs_magic));
}

__device__ __forceinline__ uint4 ld16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ bf16x8 as_frag(const uint4& r) { return __builtin_bit_cast(bf16x8, r); }

// Keeps the first `live` (0..8) bf16 of a fragment, clears the rest.
__device__ __forceinline__ uint4 keep_first(const uint4& r, int live) {
  if (!__any(live < 8)) return r;  // nearly every fragment is whole in every lane
  uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] &= 2 * e + 1 < live ? 0xffffffffu : (2 * e < live ? 0xffffu : 0u);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// max / sum over the four lanes of a row (lanes j, j+16, j+32, j+48)
__device__ __forceinline__ float row_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, KVF_WAVE));
  return fmaxf(v, __shfl_xor(v, 32, KVF_WAVE));
}
__device__ __forceinline__ float row_sum(float v) {
  v += __shfl_xor(v, 16, KVF_WAVE);
  return v + __shfl_xor(v, 32, KVF_WAVE);
}

// What a lane needs to find its operand fragments of the key block at kb.
struct Pages {
  const bf16_t* k_pages;
  const bf16_t* vt_pages;
  const int* table;
  int kvh, ctx, j16, kg;
};

// A page lookup: the table entry as loaded, and whether the key it was asked for exists.  The
// two are only combined where the page is used, so that nothing waits for the load before then;
// the lookup is issued one block before the fragment loads that need it.
struct PageRef {
  int page;
  bool asked;
  __device__ __forceinline__ bool ok(int nb) const { return asked && page >= 0 && page < nb; }
};
__device__ __forceinline__ PageRef page_of_key(const Pages& pg, const MArgs& a, int key) {
  const int blk = block_of(a, key);
  PageRef r;
  r.page = pg.table[min(blk, a.table_stride - 1)];  // always a valid address
  r.asked = key < pg.ctx && blk < a.table_stride;
  return r;
}
// Page that holds the keys of K tile t for this lane (row i = j16 is key kb + 8*(i/4) + 4*t + i%4)
__device__ __forceinline__ PageRef k_page(const Pages& pg, const MArgs& a, int kb, int t) {
  return page_of_key(pg, a, kb + 8 * (pg.j16 >> 2) + 4 * t + (pg.j16 & 3));
}
// Page of the keys kb + 8*kg + 0..7 (one page: the page size is a multiple of 8)
__device__ __forceinline__ PageRef v_page(const Pages& pg, const MArgs& a, int kb) {
  return page_of_key(pg, a, kb + 8 * pg.kg);
}

// K fragment of tile t, contraction step c, and how many of its eight elements count: none
// without a page or where the step reaches past d (head sizes that are odd multiples of 16).
// Offsets into the pages are counted in fragments of 16 bytes and fit 32 bits (the host checks).
template <int DT>
__device__ __forceinline__ uint4 k_fragment(const Pages& pg, const MArgs& a, int kb, int t, int c,
                                            const PageRef& ref, int& live) {
  const int key = kb + 8 * (pg.j16 >> 2) + 4 * t + (pg.j16 & 3);
  const int slot = key - block_of(a, key) * a.bs;
  const bool over = (DT % 2) && c == DT / 2 && pg.kg >= 2;
  const bool ok = ref.ok(a.nb) && !over;
  live = ok ? 8 : 0;
  const unsigned row = (static_cast<unsigned>(ok ? ref.page : 0) * a.KV + pg.kvh) * a.bs + slot;
  const unsigned off = row * (a.d / 8) + (over ? 0 : c * 4 + pg.kg);
  return ld16(pg.k_pages + static_cast<size_t>(off) * 8);
}
// V^T fragment of element tile dt (row i = j16 is element dt*16 + i), slots are keys
// kb + 8*kg + 0..7.  Keys at or past the context length hold whatever an earlier owner of the
// page left there: they do not count.
__device__ __forceinline__ uint4 v_fragment(const Pages& pg, const MArgs& a, int kb, int dt,
                                            const PageRef& ref, int& live) {
  const int key = kb + 8 * pg.kg;
  const int slot = key - block_of(a, key) * a.bs;
  const bool ok = ref.ok(a.nb);
  live = ok ? min(pg.ctx - key, 8) : 0;
  const unsigned row = (static_cast<unsigned>(ok ? ref.page : 0) * a.KV + pg.kvh) * a.d + dt * 16 + pg.j16;
  const unsigned off = row * (a.bs / 8) + slot / 8;
  return ld16(pg.vt_pages + static_cast<size_t>(off) * 8);
}

// The rows a lane works for: one per row tile.
template <int RT> struct Rows {
  bool ok[RT];
  int tok[RT], head[RT];
  int first[RT];       // first visible key of the row
  unsigned span[RT];   // visible keys are first .. first + span; a row that is none has first < 0
  int pos[RT];         // the row's own position; with slope2, only for kernels with BIAS
  float slope2[RT];    // the head's slope in log2 units
};

// One key block for the row tiles of a wave: scores, lazy softmax update, P * V.
// References live in log2 units: scale2 = scale * log2(e) > 0 is applied inside the exponent.
// BIAS: a score also gets its head's slope times the key's distance from the row's position;
// the scores are then brought to log2 units before the maximum is taken.
template <int DT, int RT, bool BIAS>
__device__ __forceinline__ void block_update(const bf16x8 (&kf)[2][(DT + 1) / 2], const bf16x8 (&vf)[DT],
                                             const bf16x8 (&qf)[RT][(DT + 1) / 2], const Rows<RT>& rows,
                                             int kb, int kg, bool edge, float scale_log2, float (&m_ref)[RT], float (&l_run)[RT],
                                             f32x4 (&acc)[RT][DT]) {
  constexpr int DC = (DT + 1) / 2;
  const float scale2 = BIAS ? 1.f : scale_log2;
  f32x4 s[RT][2];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      s[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DC; ++c)
        s[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][c], qf[rt][c], s[rt][t], 0, 0, 0);
    }
  // lane holds keys kb + 8*kg + 4*t + r of its row
  if (edge) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = kb + 8 * kg + 4 * t + r;
          const bool vis = static_cast<unsigned>(key - rows.first[rt]) <= rows.span[rt];
          s[rt][t][r] = vis ? s[rt][t][r] : -INFINITY;
        }
  }
  if constexpr (BIAS) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const float at0 = rows.slope2[rt] * static_cast<float>(kb + 8 * kg - rows.pos[rt]);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          s[rt][t][r] = fmaf(s[rt][t][r], scale_log2, fmaf(rows.slope2[rt], static_cast<float>(4 * t + r), at0));
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    // the scale is positive: the largest raw score is the largest scaled one
    const float bm = scale2 * fmaxf(fmaxf(fmaxf(s[rt][0][0], s[rt][0][1]), fmaxf(s[rt][0][2], s[rt][0][3])),
                                    fmaxf(fmaxf(s[rt][1][0], s[rt][1][1]), fmaxf(s[rt][1][2], s[rt][1][3])));
    if (__any(bm > m_ref[rt] + LAZY)) {
      const float m_new = fmaxf(m_ref[rt], row_max(bm));
      if (m_new != m_ref[rt]) {
        const float corr = __builtin_amdgcn_exp2f(m_ref[rt] - m_new);  // 0 from a reference of -inf
        l_run[rt] *= corr;
#pragma unroll
        for (int t = 0; t < DT; ++t) acc[rt][t] *= corr;
        m_ref[rt] = m_new;
      }
    }
    // a row that has seen no key yet has only -inf scores: any finite reference gives zeros
    const float m_use = m_ref[rt] == -INFINITY ? 0.f : m_ref[rt];
    f32x8 p;
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = __builtin_amdgcn_exp2f(fmaf(s[rt][t][r], scale2, -m_use));
        p[4 * t + r] = e;
        psum += e;
      }
    l_run[rt] += psum;  // this lane's share of the row's sum
    const bf16x8 pf = __builtin_convertvector(p, bf16x8);
#pragma unroll
    for (int t = 0; t < DT; ++t)
      acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t], pf, acc[rt][t], 0, 0, 0);
  }
}

__device__ __forceinline__ uint2 pack4(const f32x4& v, float f) {
  uint2 pk;
  pk.x = static_cast<uint32_t>(f32_to_bf16(v[0] * f)) | (static_cast<uint32_t>(f32_to_bf16(v[1] * f)) << 16);
  pk.y = static_cast<uint32_t>(f32_to_bf16(v[2] * f)) | (static_cast<uint32_t>(f32_to_bf16(v[3] * f)) << 16);
  return pk;
}

// Sets up the rows of `RT` tiles starting at `first_tile`; returns the positions they span.
template <int DT, int RT>
__device__ __forceinline__ void setup_rows(const bf16_t* q, const MArgs& a, int q0, int qlen, int start,
                                           int kvh, int first_tile, int j16, int kg, bool seq_ok,
                                           Rows<RT>& rows, bf16x8 (&qf)[RT][(DT + 1) / 2], int& pos_min,
                                           int& pos_max) {
  const int G = a.H / a.KV, D = a.d, rows_total = qlen * G;
  pos_min = 0x7fffffff;
  pos_max = -1;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = (first_tile + rt) * 16 + j16;
    rows.ok[rt] = seq_ok && row < rows_total;
    const int tok = rows.ok[rt] ? row / G : 0;
    rows.tok[rt] = tok;
    rows.head[rt] = kvh * G + (rows.ok[rt] ? row - tok * G : 0);
    {  // the row's position is below the context length, so it is its last visible key
      const int pos = start + tok;
      const int first = a.window > 0 && pos - a.window + 1 > 0 ? pos - a.window + 1 : 0;
      rows.first[rt] = rows.ok[rt] ? first : -1;
      rows.span[rt] = rows.ok[rt] ? static_cast<unsigned>(pos - first) : 0u;
      rows.pos[rt] = pos;
      rows.slope2[rt] = a.slopes && rows.ok[rt] ? a.slopes[rows.head[rt]] * LOG2E : 0.f;
    }
    if (seq_ok && (first_tile + rt) * 16 < rows_total) {
      int t_hi = ((first_tile + rt) * 16 + 15) / G;
      if (t_hi > qlen - 1) t_hi = qlen - 1;
      pos_min = min(pos_min, start + (first_tile + rt) * 16 / G);
      pos_max = max(pos_max, start + t_hi);
    }
    const bf16_t* qp = q + static_cast<size_t>(q0 + tok) * a.q_stride + rows.head[rt] * D + kg * 8;
#pragma unroll
    for (int c = 0; c < (DT + 1) / 2; ++c) {
      const bool ok = rows.ok[rt] && c * 32 + kg * 8 < D;
      qf[rt][c] = as_frag(ok ? ld16(qp + c * 32) : make_uint4(0u, 0u, 0u, 0u));
    }
  }
}

// ------------------------------------------------------------------------------------ query runs
// SHARE: the waves stage the fragments of each key block in LDS for each other; otherwise every
// wave loads all of them itself.
template <int DT, int RT, bool SHARE, bool BIAS>
__global__ __launch_bounds__(256) KVF_VGPR_FORM(DT <= 8) void attn_mfma_runs_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ vt_pages, const int* __restrict__ block_table,
    const int* __restrict__ work, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    bf16_t* __restrict__ out, MArgs a) {
  constexpr int DC = (DT + 1) / 2;
  constexpr int N_K = 2 * DC, N_FRAG = N_K + DT;          // fragments of a key block
  constexpr int FPW = (N_FRAG + WAVES - 1) / WAVES;       // fragments a wave stages per block
  // Fragments asked for two blocks ahead (two sets of staging registers) where the registers
  // that takes do not cost a wave per SIMD: measured at head size 128 with one row tile, 2,048
  // queries take 75.7 us with one set (three waves per SIMD) and 87.8 with two (two waves).
  constexpr bool DEEP = RT == 2 || DT <= 4;
  extern __shared__ uint4 frag_lds[];                     // SHARE: [2][N_FRAG][64]

  const int lane = threadIdx.x % KVF_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / KVF_WAVE);  // the same in all lanes
  const int j16 = lane % 16, kg = lane / 16;
  const int G = a.H / a.KV, D = a.d;
  // A work row names a sequence and up to two of its items (the second may be -1), which the
  // workgroup takes one after the other.
  const int wrow = a.kv_fastest ? blockIdx.y : blockIdx.x, kvh = a.kv_fastest ? blockIdx.x : blockIdx.y;
  const int seq = work[3 * wrow];
  if (seq < 0 || seq >= a.n_seqs) return;
  const int q0 = cu_q[seq], qlen = cu_q[seq + 1] - q0, ctx = ctx_lens[seq];
  const int start = ctx - qlen;
  const bool seq_ok = qlen > 0 && start >= 0;
  const Pages pg{k_pages, vt_pages, block_table + static_cast<size_t>(seq) * a.table_stride, kvh, ctx,
                 j16, kg};
  for (int part = 0; part < 2; ++part) {
  const int item = work[3 * wrow + 1 + part];
  if (item < 0) continue;
  const int wg_tile = item * WAVES * RT;

  Rows<RT> rows;
  bf16x8 qf[RT][DC];
  int pos_min, pos_max;
  setup_rows<DT, RT>(q, a, q0, qlen, start, kvh, wg_tile + wave * RT, j16, kg, seq_ok, rows, qf, pos_min,
                     pos_max);
  // key range of this wave, and of the workgroup (tiles wg_tile .. wg_tile + 4*RT - 1)
  int lo_w = 0, hi_w = -1;
  if (pos_max >= 0) {
    hi_w = pos_max < ctx - 1 ? pos_max : ctx - 1;
    if (a.window > 0 && pos_min - a.window + 1 > 0) lo_w = pos_min - a.window + 1;
  }
  int lo_g = 0, hi_g = -1;
  if (seq_ok && wg_tile * 16 < qlen * G) {
    int t_hi = ((wg_tile + WAVES * RT) * 16 - 1) / G;
    if (t_hi > qlen - 1) t_hi = qlen - 1;
    hi_g = start + t_hi < ctx - 1 ? start + t_hi : ctx - 1;
    const int p_lo = start + wg_tile * 16 / G;
    if (a.window > 0 && p_lo - a.window + 1 > 0) lo_g = p_lo - a.window + 1;
  }
  const float scale2 = a.scale * LOG2E;

  float m_ref[RT], l_run[RT];
  f32x4 acc[RT][DT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m_ref[rt] = -INFINITY;
    l_run[rt] = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  if (SHARE) {
    // fragment f of a block: K (tile f / DC, step f % DC) for f < N_K, then V^T element tiles;
    // wave w stages fragments w, w + 4, ...
    // What does not change from block to block is worked out once per fragment: the key a lane
    // reads relative to the block's start, and its offset inside a page apart from the key's slot
    // (in fragments of 16 bytes).
    // Two sets of staging registers and of page lookups, named apart (an index chosen at run
    // time would put them in scratch memory).  While the waves work on block p from LDS, the
    // fragments of block p + 1 are on their way in one set (asked for a whole block ago, put
    // into LDS at the end of this one), those of block p + 2 are asked for into the other, and
    // the pages of block p + 3 are looked up.  Lookups are issued before the fragment loads of
    // the same block: the load counter runs in order, so waiting for a lookup then does not
    // also wait for fragments that were asked for after it.
    struct Stage {
      uint4 frag[FPW];
      int live[FPW];
    };
    struct Lookup {
      PageRef page[FPW];
    };
    int key_off[FPW];
    unsigned lane_off[FPW];
    bool is_k[FPW], whole[FPW];
    const unsigned page_stride = static_cast<unsigned>(a.KV) * a.bs * (D / 8);
#pragma unroll
    for (int i = 0; i < FPW; ++i) {
      const int f = wave + i * WAVES;
      is_k[i] = f < N_K;
      if (is_k[i]) {
        const int t = f / DC, c = f % DC;
        key_off[i] = 8 * (j16 >> 2) + 4 * t + (j16 & 3);
        whole[i] = !((DT % 2) && c == DT / 2 && kg >= 2);  // a step that reaches past d
        lane_off[i] = static_cast<unsigned>(kvh) * a.bs * (D / 8) + (whole[i] ? c * 4 + kg : 0);
      } else {
        key_off[i] = 8 * kg;
        whole[i] = f < N_FRAG;
        lane_off[i] = (static_cast<unsigned>(kvh) * D + (f - N_K) * 16 + j16) * (a.bs / 8);
      }
    }
    // Every load below reads a valid address whatever the block (a key past the context reads
    // the table's last entry and page 0, and counts for nothing), so none of them sits in a
    // branch and the compiler can count them.
    auto locate = [&](int kb, Lookup& l) {
#pragma unroll
      for (int i = 0; i < FPW; ++i) l.page[i] = page_of_key(pg, a, kb + key_off[i]);
    };
    auto fetch = [&](int kb, const Lookup& l, Stage& st) {
#pragma unroll
      for (int i = 0; i < FPW; ++i) {
        const int key = kb + key_off[i];
        const unsigned slot = static_cast<unsigned>(key - block_of(a, key) * a.bs);
        const bool ok = l.page[i].ok(a.nb) && whole[i];
        st.live[i] = !ok ? 0 : is_k[i] ? 8 : min(ctx - key, 8);
        const unsigned off = __umul24(ok ? l.page[i].page : 0, page_stride) + lane_off[i] +
                             (is_k[i] ? __umul24(slot, D / 8) : slot >> 3);
        st.frag[i] = ld16((is_k[i] ? k_pages : vt_pages) + static_cast<size_t>(off) * 8);
      }
    };
    auto put = [&](int buf, const Stage& st) {
#pragma unroll
      for (int i = 0; i < FPW; ++i) {
        const int f = wave + i * WAVES;
        if (f < N_FRAG) frag_lds[(buf * N_FRAG + f) * KVF_WAVE + lane] = keep_first(st.frag[i], st.live[i]);
      }
    };
    auto work_on = [&](int kb, int buf) {
      if (kb <= hi_w && kb + 31 >= lo_w) {
        bf16x8 kf[2][DC], vf[DT];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int c = 0; c < DC; ++c)
            kf[t][c] = as_frag(frag_lds[(buf * N_FRAG + t * DC + c) * KVF_WAVE + lane]);
#pragma unroll
        for (int t = 0; t < DT; ++t) vf[t] = as_frag(frag_lds[(buf * N_FRAG + N_K + t) * KVF_WAVE + lane]);
        const bool edge = kb + 31 > pos_min || kb + 32 > ctx || a.window > 0;
        block_update<DT, RT, BIAS>(kf, vf, qf, rows, kb, kg, edge, scale2, m_ref, l_run, acc);
      }
    };
    const int kb_first = (lo_g / 32) * 32;
    Stage sa;
    Lookup la;
    if constexpr (DEEP) {
      Stage sb;
      Lookup lb;
      if (kb_first <= hi_g) {
        locate(kb_first, la);
        locate(kb_first + 32, lb);
        fetch(kb_first, la, sa);
        locate(kb_first + 64, la);
        fetch(kb_first + 32, lb, sb);
        put(0, sa);
      }
      // Everything loaded so far (the query fragments among it) has to be there before the loop:
      // otherwise the compiler, not knowing how many loads a first pass through the loop still
      // has ahead of them, waits for all loads before the first product of every pass.
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      __syncthreads();
      // at the top of a pass: LDS half 0 holds block kb, `sb` block kb + 32, `la` the pages of
      // block kb + 64
      for (int kb = kb_first; kb <= hi_g; kb += 64) {
        locate(kb + 96, lb);
        fetch(kb + 64, la, sa);
        work_on(kb, 0);
        put(1, sb);
        __syncthreads();
        if (kb + 32 > hi_g) break;
        locate(kb + 128, la);
        fetch(kb + 96, lb, sb);
        work_on(kb + 32, 1);
        put(0, sa);
        __syncthreads();
      }
    } else {
      // one set: the fragments of block p + 1 are asked for at the top of block p and put into
      // LDS at its end; the pages of block p + 2 are looked up meanwhile
      if (kb_first <= hi_g) {
        locate(kb_first, la);
        fetch(kb_first, la, sa);
        locate(kb_first + 32, la);
        put(0, sa);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), as above
      __syncthreads();
      int buf = 0;
      for (int kb = kb_first; kb <= hi_g; kb += 32) {
        fetch(kb + 32, la, sa);
        locate(kb + 64, la);
        work_on(kb, buf);
        put(buf ^ 1, sa);
        __syncthreads();
        buf ^= 1;
      }
    }
  } else {
    PageRef pk[2] = {k_page(pg, a, (lo_w / 32) * 32, 0), k_page(pg, a, (lo_w / 32) * 32, 1)};
    PageRef pv = v_page(pg, a, (lo_w / 32) * 32);
    for (int kb = (lo_w / 32) * 32; kb <= hi_w; kb += 32) {
      uint4 kr[2][DC], vr[DT];
      int kl[2][DC], vl;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c = 0; c < DC; ++c) kr[t][c] = k_fragment<DT>(pg, a, kb, t, c, pk[t], kl[t][c]);
#pragma unroll
      for (int t = 0; t < DT; ++t) vr[t] = v_fragment(pg, a, kb, t, pv, vl);
      pk[0] = k_page(pg, a, kb + 32, 0);
      pk[1] = k_page(pg, a, kb + 32, 1);
      pv = v_page(pg, a, kb + 32);
      bf16x8 kf[2][DC], vf[DT];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c = 0; c < DC; ++c) kf[t][c] = as_frag(keep_first(kr[t][c], kl[t][c]));
#pragma unroll
      for (int t = 0; t < DT; ++t) vf[t] = as_frag(keep_first(vr[t], vl));
      const bool edge = kb + 31 > pos_min || kb + 32 > ctx || a.window > 0;
      block_update<DT, RT, BIAS>(kf, vf, qf, rows, kb, kg, edge, scale2, m_ref, l_run, acc);
    }
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float l = row_sum(l_run[rt]);
    if (!rows.ok[rt]) continue;
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16_t* o = out + static_cast<size_t>(q0 + rows.tok[rt]) * a.o_stride + rows.head[rt] * D + 4 * kg;
#pragma unroll
    for (int t = 0; t < DT; ++t) *reinterpret_cast<uint2*>(o + t * 16) = pack4(acc[rt][t], inv);
  }
  __syncthreads();  // the staging buffers are free for the next item
  }  // part
}

// ------------------------------------------------------------------------- few rows, split keys
// TWO: a wave holds the fragments of two blocks, loading one while it consumes the other.
// NW: waves of the workgroup; more of them shorten each wave's walk over its cut of the keys.
template <int DT, bool TWO, int NW, bool BIAS>
__global__ __launch_bounds__(NW * KVF_WAVE) KVF_VGPR_FORM(DT <= 6) void attn_mfma_split_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ vt_pages, const int* __restrict__ block_table,
    const int* __restrict__ seq_ids, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    bf16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml, MArgs a) {
  constexpr int DC = (DT + 1) / 2;
  extern __shared__ float lds[];  // [NW][DT][64][4] accumulators, then [NW][16][2]

  const int lane = threadIdx.x % KVF_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / KVF_WAVE);  // the same in all lanes
  const int j16 = lane % 16, kg = lane / 16;
  const int G = a.H / a.KV, D = a.d;
  const int chunks = (G + 15) / 16;
  // The kv heads are the fastest index of the grid: consecutive workgroups go to different
  // XCDs, so the heads of one sequence pull on the cache through all of them, however its
  // context compares with the others' (with the sequences in front, all workgroups of a sequence
  // whose index is fixed modulo 8 landed on one XCD, and one long context among short ones was
  // read through an eighth of the chip).
  const int entry = blockIdx.y;
  const int seq = seq_ids ? seq_ids[entry] : entry;
  if (seq < 0 || seq >= a.n_seqs) return;
  const int kvh = blockIdx.x / chunks, tile = blockIdx.x - kvh * chunks;
  // without cu_q every sequence has one token, its own: nothing then waits for a load before the
  // query and the page lookups can be asked for
  const int q0 = cu_q ? cu_q[seq] : seq, qlen = cu_q ? cu_q[seq + 1] - q0 : 1, ctx = ctx_lens[seq];
  const int start = ctx - qlen;
  const bool seq_ok = qlen > 0 && start >= 0;
  const Pages pg{k_pages, vt_pages, block_table + static_cast<size_t>(seq) * a.table_stride, kvh, ctx,
                 j16, kg};
  Rows<1> rows;
  bf16x8 qf[1][DC];
  int pos_min, pos_max;
  setup_rows<DT, 1>(q, a, q0, qlen, start, kvh, tile, j16, kg, seq_ok, rows, qf, pos_min, pos_max);
  int lo = 0, hi = -1;
  if (pos_max >= 0) {
    hi = pos_max < ctx - 1 ? pos_max : ctx - 1;
    if (a.window > 0 && pos_min - a.window + 1 > 0) lo = pos_min - a.window + 1;
  }
  // Blocks of 32 keys go round the waves of all cuts in turn: cut z, wave w take blocks
  // z * NW + w, then every (NW * splits)-th.  Without a window the first block is known before
  // the context length has arrived.
  const int kb0 = (lo / 32) * 32;
  const int kb_end = hi + 1;
  const int turn = (static_cast<int>(blockIdx.z) * NW + wave) * 32;
  const int kb_begin = kb0 + turn;
  const int STEP = 32 * NW * a.splits;
  const float scale2 = a.scale * LOG2E;

  float m_ref[1] = {-INFINITY}, l_run[1] = {0.f};
  f32x4 acc[1][DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) acc[0][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // The register buffers are named apart (an index chosen at run time would put them in
  // scratch); the pages of a block are looked up one block before its fragments are loaded.
  struct Raw {
    uint4 k[2][DC], v[DT];
    int kl[2][DC], vl;
  };
  Raw A, B;
  PageRef pA[3], pB[3];
  auto locate = [&](int kb, PageRef (&p)[3]) {
    p[0] = k_page(pg, a, kb, 0);
    p[1] = k_page(pg, a, kb, 1);
    p[2] = v_page(pg, a, kb);
  };
  auto fetch = [&](int kb, const PageRef (&p)[3], Raw& r) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int c = 0; c < DC; ++c) r.k[t][c] = k_fragment<DT>(pg, a, kb, t, c, p[t], r.kl[t][c]);
#pragma unroll
    for (int t = 0; t < DT; ++t) r.v[t] = v_fragment(pg, a, kb, t, p[2], r.vl);
  };
  auto consume = [&](int kb, const Raw& r) {
    bf16x8 kf[2][DC], vf[DT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int c = 0; c < DC; ++c) kf[t][c] = as_frag(keep_first(r.k[t][c], r.kl[t][c]));
#pragma unroll
    for (int t = 0; t < DT; ++t) vf[t] = as_frag(keep_first(r.v[t], r.vl));
    const bool edge = kb + 31 > pos_min || kb + 32 > ctx || a.window > 0;
    block_update<DT, 1, BIAS>(kf, vf, qf, rows, kb, kg, edge, scale2, m_ref, l_run, acc);
  };
  // Without a window the page lookups of the first blocks are asked for together with the
  // query and the context length, not after them: one round trip to memory less.
  const bool early = a.window <= 0;
  if (early) {
    locate(turn, pA);
    if (TWO) locate(turn + STEP, pB);
  }
  // the query fragments have to be there before the loops (see the note in the runs kernel)
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  if (TWO) {
    if (kb_begin < kb_end) {
      if (!early) {
        locate(kb_begin, pA);
        locate(kb_begin + STEP, pB);
      }
      fetch(kb_begin, pA, A);
    }
    for (int kb = kb_begin; kb < kb_end; kb += 2 * STEP) {
      const bool second = kb + STEP < kb_end;
      if (second) fetch(kb + STEP, pB, B);
      locate(kb + 2 * STEP, pA);
      consume(kb, A);
      if (second) {
        if (kb + 2 * STEP < kb_end) fetch(kb + 2 * STEP, pA, A);
        locate(kb + 3 * STEP, pB);
        consume(kb + STEP, B);
      }
    }
  } else {
    if (!early) locate(kb_begin, pA);
    for (int kb = kb_begin; kb < kb_end; kb += STEP) {
      fetch(kb, pA, A);
      locate(kb + STEP, pA);
      consume(kb, A);
    }
  }

  // ---- merge the waves, then store or hand on the partial result
  float* red_acc = lds;                             // [NW][DT][64][4]
  float* red_ml = lds + NW * DT * KVF_WAVE * 4;  // [NW][16][2]
  const float l_row = row_sum(l_run[0]);
#pragma unroll
  for (int t = 0; t < DT; ++t)
    *reinterpret_cast<f32x4*>(red_acc + ((wave * DT + t) * KVF_WAVE + lane) * 4) = acc[0][t];
  if (kg == 0) {
    red_ml[(wave * 16 + j16) * 2] = m_ref[0];
    red_ml[(wave * 16 + j16) * 2 + 1] = l_row;
  }
  __syncthreads();
  float mm = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) mm = fmaxf(mm, red_ml[(w * 16 + j16) * 2]);
  float cw[NW], ll = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float mw = red_ml[(w * 16 + j16) * 2];
    cw[w] = mw == -INFINITY ? 0.f : exp2f(mw - mm);
    ll += red_ml[(w * 16 + j16) * 2 + 1] * cw[w];
  }
  if (a.splits == 1 && qlen == 1 && ctx <= 0) {
    // a sequence without context (the padding of a captured batch): a row of zeros, as the merge
    // of cuts gives it, so that no row of the output keeps what an earlier step left there
    const int g = tile * 16 + j16;
    if (g < G)
      for (int t = wave; t < DT; t += NW)
        *reinterpret_cast<uint2*>(out + static_cast<size_t>(q0) * a.o_stride + (kvh * G + g) * D + t * 16 +
                                  4 * kg) = make_uint2(0u, 0u);
    return;
  }
  if (!rows.ok[0]) return;
  const int head = rows.head[0];
  const size_t slot = (static_cast<size_t>(entry) * a.H + head) * a.splits + blockIdx.z;
  if (a.splits > 1 && wave == 0 && kg == 0) {
    part_ml[slot * 2] = mm;  // in log2 units
    part_ml[slot * 2 + 1] = ll;
  }
  const float inv = ll > 0.f ? 1.f / ll : 0.f;
  for (int t = wave; t < DT; t += NW) {  // wave w finishes element tiles w, w + NW, ...
    f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < NW; ++w)
      o += *reinterpret_cast<const f32x4*>(red_acc + ((w * DT + t) * KVF_WAVE + lane) * 4) * cw[w];
    const int e0 = t * 16 + 4 * kg;
    if (a.splits == 1)
      *reinterpret_cast<uint2*>(out + static_cast<size_t>(q0 + rows.tok[0]) * a.o_stride + head * D + e0) =
          pack4(o, inv);
    else
      *reinterpret_cast<f32x4*>(part_acc + slot * D + e0) = o;
  }
}

// Merges the splits of every (sequence, head) in split order.  One query token per sequence, one
// wave per (sequence, head), at most 64 splits; the partial maxima are in log2 units.  Lane s
// weighs split s; the loads of the partial accumulators do not depend on one another.  A
// sequence without context (the padding of a captured batch) has no partial results: its row
// is cleared and the workspace is not read.
__global__ __launch_bounds__(64) void attn_split_combine_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    const int* __restrict__ seq_ids, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    bf16_t* __restrict__ out, int H, int D, int splits, int o_stride, int n_seqs) {
  const int seq = seq_ids ? seq_ids[blockIdx.x] : static_cast<int>(blockIdx.x);
  if (seq < 0 || seq >= n_seqs) return;
  const int head = blockIdx.y, lane = threadIdx.x;
  if (ctx_lens[seq] <= 0) {
    const int token = cu_q ? cu_q[seq] : seq;
    for (int e = lane; e < D; e += KVF_WAVE) out[static_cast<size_t>(token) * o_stride + head * D + e].bits = 0;
    return;
  }
  const size_t slot0 = (static_cast<size_t>(blockIdx.x) * H + head) * splits;
  float m = -INFINITY, l = 0.f;
  if (lane < splits) {
    const float2 ml = *reinterpret_cast<const float2*>(part_ml + (slot0 + lane) * 2);
    m = ml.x;
    l = ml.y;
  }
  const int tok = cu_q ? cu_q[seq] : seq;
  const float mm = wave_max(m);
  const float c = m == -INFINITY ? 0.f : exp2f(m - mm);
  const float ll = wave_sum(l * c);
  const float inv = ll > 0.f ? 1.f / ll : 0.f;
  for (int e = lane; e < D; e += KVF_WAVE) {
    float v = 0.f;
#pragma unroll 8
    for (int s = 0; s < splits; ++s)
      v += part_acc[(slot0 + s) * D + e] *
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, c), s));
    out[static_cast<size_t>(tok) * o_stride + head * D + e].bits = f32_to_bf16(v * inv);
  }
}

// Also what the 32-bit arithmetic in the kernels needs: positions * page size and the number of
// 16-byte fragments of a page tensor below 2^32.
bool args_ok(int H, int KV, int d, int bs, int nb, int table_stride, float scale) {
  if (!(d > 0 && d % 16 == 0 && d <= 256 && KV > 0 && H % KV == 0 && bs > 0 && bs % 8 == 0)) return false;
  if (nb < 1 || table_stride < 1 || !(scale > 0.f)) return false;
  const unsigned long long limit = 1ull << 32;
  // (the page number and a page's size in fragments also go through 24-bit multiplies)
  return static_cast<unsigned long long>(table_stride) * bs * bs < limit &&
         static_cast<unsigned long long>(nb) * KV * bs * d / 8 < limit && nb < (1 << 24) &&
         static_cast<unsigned long long>(KV) * bs * d / 8 < (1ull << 24);
}
unsigned magic_of(int bs) { return static_cast<unsigned>((1ull << 32) / bs) + 1u; }

// Row tiles per wave and LDS sharing by head size: what fits the registers and 64 KB of LDS.
// One tile per wave keeps more workgroups in flight; two halve what a key block costs per row
// (looking its pages up, staging it, the barrier) and pay when the work fills the chip anyway
// (measured at 32 heads of size 64, one item per workgroup: 8,192 tokens 444 to 385 us, 4,096
// tokens 143 to 114; 2,048 tokens 47 to 54 the other way): the caller chooses by the rows it
// has and by kvf_attn_mfma_prefill_blocks_per_cu.
constexpr int runs_max_rt(int dt) { return dt <= 8 ? 2 : 1; }
constexpr bool runs_share(int dt) { return dt <= 12; }

template <int DT, int RT>
void launch_runs_rt(dim3 grid, hipStream_t s, const void* q, const void* k_pages, const void* vt_pages,
                    const int* block_table, const int* work, const int* cu_q, const int* ctx_lens, void* out,
                    const MArgs& a) {
  constexpr bool SHARE = runs_share(DT);
  constexpr int N_FRAG = 2 * ((DT + 1) / 2) + DT;
  const size_t lds = SHARE ? static_cast<size_t>(2) * N_FRAG * KVF_WAVE * sizeof(uint4) : 0;
  if (a.slopes)
    hipLaunchKernelGGL((attn_mfma_runs_kernel<DT, RT, SHARE, true>), grid, dim3(256), lds, s,
                       static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),
                       static_cast<const bf16_t*>(vt_pages), block_table, work, cu_q, ctx_lens,
                       static_cast<bf16_t*>(out), a);
  else
    hipLaunchKernelGGL((attn_mfma_runs_kernel<DT, RT, SHARE, false>), grid, dim3(256), lds, s,
                       static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),
                       static_cast<const bf16_t*>(vt_pages), block_table, work, cu_q, ctx_lens,
                       static_cast<bf16_t*>(out), a);
}

template <int DT>
void launch_runs(int row_tiles, dim3 grid, hipStream_t s, const void* q, const void* k_pages,
                 const void* vt_pages, const int* block_table, const int* work, const int* cu_q,
                 const int* ctx_lens, void* out, const MArgs& a) {
  if constexpr (runs_max_rt(DT) >= 2) {
    if (row_tiles == 2) {
      launch_runs_rt<DT, 2>(grid, s, q, k_pages, vt_pages, block_table, work, cu_q, ctx_lens, out, a);
      return;
    }
  }
  launch_runs_rt<DT, 1>(grid, s, q, k_pages, vt_pages, block_table, work, cu_q, ctx_lens, out, a);
}

template <int DT, int NW>
void launch_split_waves(dim3 grid, hipStream_t s, const void* q, const void* k_pages, const void* vt_pages,
                        const int* block_table, const int* seq_ids, const int* cu_q, const int* ctx_lens,
                        void* out, float* part_acc, float* part_ml, const MArgs& a) {
  const size_t lds = (static_cast<size_t>(NW) * DT * KVF_WAVE * 4 + NW * 16 * 2) * sizeof(float);
  if (a.slopes)
    hipLaunchKernelGGL((attn_mfma_split_kernel<DT, (DT <= 8), NW, true>), grid, dim3(NW * KVF_WAVE), lds, s,
                       static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),
                       static_cast<const bf16_t*>(vt_pages), block_table, seq_ids, cu_q, ctx_lens,
                       static_cast<bf16_t*>(out), part_acc, part_ml, a);
  else
    hipLaunchKernelGGL((attn_mfma_split_kernel<DT, (DT <= 8), NW, false>), grid, dim3(NW * KVF_WAVE), lds, s,
                       static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),
                       static_cast<const bf16_t*>(vt_pages), block_table, seq_ids, cu_q, ctx_lens,
                       static_cast<bf16_t*>(out), part_acc, part_ml, a);
}

int g_split_waves = 0;  // measurement aid: 4 or 8 waves per workgroup, 0 = by the grid

// Eight waves shorten each wave's walk over the keys when the grid leaves compute units idle
// anyway (and two blocks of fragments still fit the registers that leaves each wave); a grid
// that fills the chip does better with four.
template <int DT>
void launch_split(dim3 grid, hipStream_t s, const void* q, const void* k_pages, const void* vt_pages,
                  const int* block_table, const int* seq_ids, const int* cu_q, const int* ctx_lens,
                  void* out, float* part_acc, float* part_ml, const MArgs& a) {
  const size_t groups = static_cast<size_t>(grid.x) * grid.y * grid.z;
  const bool eight = g_split_waves ? g_split_waves == 8 : groups <= 256;
  if (DT <= 6 && eight)
    launch_split_waves<DT, (DT <= 6 ? 8 : 4)>(grid, s, q, k_pages, vt_pages, block_table, seq_ids, cu_q,
                                              ctx_lens, out, part_acc, part_ml, a);
  else
    launch_split_waves<DT, 4>(grid, s, q, k_pages, vt_pages, block_table, seq_ids, cu_q, ctx_lens, out,
                              part_acc, part_ml, a);
}

#define KVF_EACH_DT(X) \
  X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15) X(16)
}  // namespace

// For measurements: waves per workgroup of the kernel for single tokens (4, 8; 0 = by the grid).
KVF_EXPORT void kvf_attn_mfma_set_split_waves(int waves) { g_split_waves = waves; }
// Rows of a query run one workgroup takes with `row_tiles` (1 or 2) tiles per wave, where the
// head size allows so many: 4 waves x tiles x 16 rows.
KVF_EXPORT int kvf_attn_mfma_rows_per_item(int d, int row_tiles) {
  const int most = d > 0 && d <= 128 ? 2 : 1;   // runs_max_rt(d / 16)
  return WAVES * (row_tiles >= 2 ? most : 1) * 16;
}

// Workgroups of the kernel for query runs that a compute unit holds at once, by its registers
// and LDS: what a caller weighs rows per item against (0 if the head size is not taken).
template <int DT, int RT>
int runs_blocks_per_cu() {
  constexpr bool SHARE = runs_share(DT);
  constexpr int N_FRAG = 2 * ((DT + 1) / 2) + DT;
  const size_t lds = SHARE ? static_cast<size_t>(2) * N_FRAG * KVF_WAVE * sizeof(uint4) : 0;
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, attn_mfma_runs_kernel<DT, RT, SHARE, false>, 256, lds) !=
      hipSuccess)
    return 0;
  return n;
}
KVF_EXPORT int kvf_attn_mfma_prefill_blocks_per_cu(int d, int row_tiles) {
  if (d <= 0 || d % 16 != 0 || d > 256) return 0;
  const bool two = row_tiles >= 2 && d <= 128;
  switch (d / 16) {
#define GO(DT)                                                              \
  case DT:                                                                  \
    if constexpr (runs_max_rt(DT) >= 2) {                                   \
      if (two) return runs_blocks_per_cu<DT, 2>();                          \
    }                                                                       \
    return runs_blocks_per_cu<DT, 1>();
    KVF_EACH_DT(GO)
#undef GO
  }
  return 0;
}

// Query runs: `work` holds num_work rows (sequence, item, item or -1) where item i covers rows
// [i * rows_per_item, (i + 1) * rows_per_item) of the sequence's qlen * H/KV rows per kv head;
// rows_per_item is what kvf_attn_mfma_rows_per_item gave for one or two row tiles.
KVF_EXPORT int kvf_attn_mfma_prefill(const void* q, const void* k_pages, const void* vt_pages,
                                     const int* block_table, const int* cu_q, const int* ctx_lens,
                                     const int* work, int num_work, int rows_per_item, void* out, int H, int KV, int d,
                                     int bs, int nb, int table_stride, int q_stride, int o_stride,
                                     int window, int n_seqs, float scale, const float* slopes,
                                     hipStream_t s) {
  if (num_work <= 0) return 0;
  if (!args_ok(H, KV, d, bs, nb, table_stride, scale) || q_stride % 8 != 0 || o_stride % 4 != 0)
    return static_cast<int>(hipErrorInvalidValue);
  const int row_tiles = rows_per_item / (WAVES * 16);
  if (rows_per_item != kvf_attn_mfma_rows_per_item(d, row_tiles)) return static_cast<int>(hipErrorInvalidValue);
  // The kv heads are the fastest index of the grid where the grid allows it: consecutive
  // workgroups go to consecutive XCDs, so with eight kv heads every XCD walks the keys and values
  // of one head and finds them in its own L2 after the first workgroup has brought them in.
  const int kv_fastest = num_work <= 65535 ? 1 : 0;
  const MArgs a{H, KV, d, bs, nb, table_stride, q_stride, o_stride, window, n_seqs, 1, kv_fastest, scale, magic_of(bs), slopes};
  const dim3 grid = kv_fastest ? dim3(KV, num_work) : dim3(num_work, KV);
  switch (d / 16) {
#define GO(DT) \
  case DT: launch_runs<DT>(row_tiles, grid, s, q, k_pages, vt_pages, block_table, work, cu_q, ctx_lens, out, a); break;
    KVF_EACH_DT(GO)
#undef GO
  }
  return kvf_last_error();
}

// Single-token queries: sequences seq_ids[0..num_seqs) (or 0..num_seqs-1), key range cut into
// `splits`.  cu_q may be null when the token of sequence i is token i.  With splits > 1, part_acc holds num_seqs*H*splits*d floats and part_ml
// num_seqs*H*splits*2; calls that share them must not overlap.
KVF_EXPORT int kvf_attn_mfma_decode(const void* q, const void* k_pages, const void* vt_pages,
                                    const int* block_table, const int* seq_ids, const int* cu_q,
                                    const int* ctx_lens, void* out, float* part_acc, float* part_ml,
                                    int num_seqs, int H, int KV, int d, int bs, int nb,
                                    int table_stride, int q_stride, int o_stride, int window,
                                    int n_seqs, int splits, float scale, const float* slopes,
                                    hipStream_t s) {
  if (num_seqs <= 0) return 0;
  if (!args_ok(H, KV, d, bs, nb, table_stride, scale) || q_stride % 8 != 0 || o_stride % 4 != 0 || splits < 1 ||
      splits > KVF_WAVE || (splits > 1 && (!part_acc || !part_ml)))
    return static_cast<int>(hipErrorInvalidValue);
  const MArgs a{H, KV, d, bs, nb, table_stride, q_stride, o_stride, window, n_seqs, splits, 0, scale, magic_of(bs), slopes};
  const int G = H / KV, chunks = (G + 15) / 16;
  if (num_seqs > 65535) return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid(KV * chunks, num_seqs, splits);
  switch (d / 16) {
#define GO(DT)                                                                                      \
  case DT:                                                                                          \
    launch_split<DT>(grid, s, q, k_pages, vt_pages, block_table, seq_ids, cu_q, ctx_lens, out, part_acc, \
                     part_ml, a);                                                                   \
    break;
    KVF_EACH_DT(GO)
#undef GO
  }
  int err = kvf_last_error();
  if (err || splits == 1) return err;
  hipLaunchKernelGGL(attn_split_combine_kernel, dim3(num_seqs, H), dim3(64), 0, s, part_acc,
                     part_ml, seq_ids, cu_q, ctx_lens, static_cast<bf16_t*>(out), H, d, splits,
                     o_stride, n_seqs);
  return kvf_last_error();
}
