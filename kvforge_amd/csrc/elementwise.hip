// Row-wise kernels of the decoder: embedding gather, RMS norm, SwiGLU gate, rotary + cache write.
// The residual stream is fp32 in every mode; T is the activation / weight element type.
#include "common.h"

// ----------------------------------------------------------------------------- embedding
// out[n, :] = table[ids[n], :] widened to fp32.  An id outside [0, vocab) writes zeros.
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ out, int h, int vocab) {
  const int n = blockIdx.x;
  const int id = ids[n];
  float* o = out + static_cast<size_t>(n) * h;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < h; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* row = table + static_cast<size_t>(id) * h;
  for (int i = threadIdx.x; i < h; i += blockDim.x) o[i] = Elem<T>::load(row + i);
}

template <typename T>
static int embed_launch(const int* ids, const void* table, float* out, int n, int h, int vocab,
                        hipStream_t s) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(embed_kernel<T>, dim3(n), dim3(256), 0, s, ids, static_cast<const T*>(table),
                     out, h, vocab);
  return kvf_last_error();
}
KVF_EXPORT int kvf_embed_f32(const int* ids, const void* t, float* o, int n, int h, int v,
                             hipStream_t s) { return embed_launch<float>(ids, t, o, n, h, v, s); }
KVF_EXPORT int kvf_embed_bf16(const int* ids, const void* t, float* o, int n, int h, int v,
                              hipStream_t s) { return embed_launch<bf16_t>(ids, t, o, n, h, v, s); }

// ----------------------------------------------------------------------------- RMS norm
// y = x * rsqrt(mean(x^2) + eps) * w, all in fp32, rounded once to T on store.
// x is the fp32 residual stream; `rows` (may be null) gathers input rows; w is fp32 or T, or
// null when the weight has been folded into the matrix that consumes y.
// `delta` (may be null, [x_rows, h] of T) is a sum still owed to the stream: the norm is taken of
// x + delta, and without `rows` the sum is also written back to x, which saves the pass of an
// add kernel of its own.
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                     __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u));
}
__device__ __forceinline__ void store4(float* p, const float4& v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, const float4& v) {
  uint2 r;
  r.x = static_cast<uint32_t>(f32_to_bf16(v.x)) | (static_cast<uint32_t>(f32_to_bf16(v.y)) << 16);
  r.y = static_cast<uint32_t>(f32_to_bf16(v.z)) | (static_cast<uint32_t>(f32_to_bf16(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = r;
}

constexpr int NORM_KEEP = 4;  // float4s a thread keeps in registers between the two passes

template <typename T, typename W, typename D>
__global__ void rmsnorm_kernel(float* __restrict__ x, const int* __restrict__ rows,
                               const D* __restrict__ delta, const W* __restrict__ w, float eps,
                               T* __restrict__ out, int h, int x_rows, int aligned) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  int src = rows ? rows[m] : m;
  T* o = out + static_cast<size_t>(m) * h;
  if (src < 0 || src >= x_rows) {
    for (int i = threadIdx.x; i < h; i += blockDim.x) Elem<T>::store(o + i, 0.f);
    return;
  }
  float* xr = x + static_cast<size_t>(src) * h;
  const D* dr = delta ? delta + static_cast<size_t>(src) * h : nullptr;
  const bool write_back = dr && !rows;
  float ss = 0.f;
  if (aligned && h <= static_cast<int>(blockDim.x) * 4 * NORM_KEEP) {
    // the row stays in registers: one read of x (and delta), one write of y (and x)
    float4 v[NORM_KEEP];
#pragma unroll
    for (int k = 0; k < NORM_KEEP; ++k) {
      const int i = (k * blockDim.x + threadIdx.x) * 4;
      v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < h) {
        v[k] = load4(xr + i);
        if (dr) {
          const float4 d = load4(dr + i);
          v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w;
          if (write_back) store4(xr + i, v[k]);
        }
        ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
      }
    }
    ss = block_sum(ss, scratch);
    const float r = rsqrtf(ss / static_cast<float>(h) + eps);
#pragma unroll
    for (int k = 0; k < NORM_KEEP; ++k) {
      const int i = (k * blockDim.x + threadIdx.x) * 4;
      if (i < h) {
        float4 y = make_float4(v[k].x * r, v[k].y * r, v[k].z * r, v[k].w * r);
        if (w) {
          const float4 g = load4(w + i);
          y.x *= g.x; y.y *= g.y; y.z *= g.z; y.w *= g.w;
        }
        store4(o + i, y);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = xr[i];
    if (dr) {
      v += Elem<D>::load(dr + i);
      if (write_back) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = rsqrtf(ss / static_cast<float>(h) + eps);
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = xr[i];  // already the sum where it was written back (by this same thread)
    if (dr && !write_back) v += Elem<D>::load(dr + i);
    Elem<T>::store(o + i, w ? v * r * Elem<W>::load(w + i) : v * r);
  }
}

template <typename T, typename D>
static int rmsnorm_launch(float* x, const int* rows, const void* delta, const void* w, int w_is_f32,
                          float eps, void* out, int m, int h, int x_rows, hipStream_t s) {
  if (m <= 0) return 0;
  const int threads = h >= 1024 ? 256 : (h >= 256 ? 128 : 64);
  auto at = [](const void* p, size_t a) { return reinterpret_cast<uintptr_t>(p) % a == 0; };
  const int aligned = h % 4 == 0 && at(x, 16) && at(out, 4 * sizeof(T)) && at(delta, 4 * sizeof(D)) &&
                      at(w, w_is_f32 ? 16 : 4 * sizeof(T));
  if (w_is_f32)
    hipLaunchKernelGGL((rmsnorm_kernel<T, float, D>), dim3(m), dim3(threads), 0, s, x, rows,
                       static_cast<const D*>(delta), static_cast<const float*>(w), eps,
                       static_cast<T*>(out), h, x_rows, aligned);
  else
    hipLaunchKernelGGL((rmsnorm_kernel<T, T, D>), dim3(m), dim3(threads), 0, s, x, rows,
                       static_cast<const D*>(delta), static_cast<const T*>(w), eps,
                       static_cast<T*>(out), h, x_rows, aligned);
  return kvf_last_error();
}
// delta (may be null): a sum still owed to x, in the type of `out` or (delta_f32) in fp32
KVF_EXPORT int kvf_rmsnorm_f32(float* x, const int* rows, const void* delta, int delta_f32, const void* w,
                               int wf, float eps, void* out, int m, int h, int xr, hipStream_t s) {
  (void)delta_f32;
  return rmsnorm_launch<float, float>(x, rows, delta, w, wf, eps, out, m, h, xr, s);
}
KVF_EXPORT int kvf_rmsnorm_bf16(float* x, const int* rows, const void* delta, int delta_f32, const void* w,
                                int wf, float eps, void* out, int m, int h, int xr, hipStream_t s) {
  if (delta_f32) return rmsnorm_launch<bf16_t, float>(x, rows, delta, w, wf, eps, out, m, h, xr, s);
  return rmsnorm_launch<bf16_t, bf16_t>(x, rows, delta, w, wf, eps, out, m, h, xr, s);
}

// ----------------------------------------------------------------------------- residual sum
// x[m] += delta[m] in fp32 (x is the residual stream, delta a product in T).
template <typename T>
__global__ void add_rows_kernel(float* __restrict__ x, const T* __restrict__ delta, size_t total) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) x[i] += Elem<T>::load(delta + i);
}
template <typename T>
static int add_rows_launch(float* x, const void* delta, int m, int h, hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * h;
  if (total == 0) return 0;
  hipLaunchKernelGGL(add_rows_kernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, s,
                     x, static_cast<const T*>(delta), total);
  return kvf_last_error();
}
KVF_EXPORT int kvf_add_rows_f32(float* x, const void* d, int m, int h, hipStream_t s) {
  return add_rows_launch<float>(x, d, m, h, s);
}
KVF_EXPORT int kvf_add_rows_bf16(float* x, const void* d, int m, int h, hipStream_t s) {
  return add_rows_launch<bf16_t>(x, d, m, h, s);
}

// ----------------------------------------------------------------------------- SwiGLU gate
// out[m, i] = silu(gate) * up with silu(x) = x / (1 + exp(-x)), in fp32.  The input row holds
// gate and up side by side: gate at 2i and up at 2i + 1 (`paired` != 0, the layout the fused
// gate/up matrix produces) or gate at i and up at I + i.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter,
                                size_t total, int paired) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / inter;
  const int i = static_cast<int>(idx - m * inter);
  const T* row = gu + m * 2 * static_cast<size_t>(inter);
  const float g = Elem<T>::load(paired ? row + 2 * i : row + i);
  const float u = Elem<T>::load(paired ? row + 2 * i + 1 : row + inter + i);
  Elem<T>::store(out + idx, g / (1.f + expf(-g)) * u);
}
// bf16, paired: a thread takes four neighbouring (gate, up) pairs (16 bytes in, 8 bytes out)
__global__ void silu_mul_pairs4_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out,
                                       size_t quads) {
  const size_t q = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (q >= quads) return;
  float v[8];
  load8(gu + q * 8, v);
  uint2 packed;
  uint32_t h[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) h[i] = f32_to_bf16(v[2 * i] / (1.f + __expf(-v[2 * i])) * v[2 * i + 1]);
  packed.x = h[0] | (h[1] << 16);
  packed.y = h[2] | (h[3] << 16);
  *reinterpret_cast<uint2*>(out + q * 4) = packed;
}

template <typename T>
static int silu_mul_launch(const void* gu, void* out, int m, int inter, int paired,
                           hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * inter;
  if (total == 0) return 0;
  if (sizeof(T) == 2 && paired && inter % 4 == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 8 == 0) {
    const size_t quads = total / 4;
    hipLaunchKernelGGL(silu_mul_pairs4_kernel, dim3(static_cast<unsigned>((quads + 255) / 256)), dim3(256),
                       0, s, static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), quads);
    return kvf_last_error();
  }
  const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
  hipLaunchKernelGGL(silu_mul_kernel<T>, dim3(blocks), dim3(256), 0, s,
                     static_cast<const T*>(gu), static_cast<T*>(out), inter, total, paired);
  return kvf_last_error();
}
KVF_EXPORT int kvf_silu_mul_f32(const void* gu, void* out, int m, int inter, int paired,
                                hipStream_t s) {
  return silu_mul_launch<float>(gu, out, m, inter, paired, s);
}
KVF_EXPORT int kvf_silu_mul_bf16(const void* gu, void* out, int m, int inter, int paired,
                                 hipStream_t s) {
  return silu_mul_launch<bf16_t>(gu, out, m, inter, paired, s);
}

// ----------------------------------------------------------------------------- rotary + cache write
// qkv: [N, (H + 2*KV) * d] rows of q heads, then k heads, then v heads.
// A rotary pair is two neighbouring elements (2i, 2i + 1) of a head: the projection matrices
// are stored with their rows permuted so that what the checkpoint's layout calls elements i and
// i + rot/2 land there (a dot product of q and k does not care about the order, and v and the
// output projection are not permuted).  For token n at position p (cos/sin tables
// [table_len, rot/2] fp32) and i < rot/2:
//   x'[2i] = x[2i]*cos[i] - x[2i+1]*sin[i];   x'[2i+1] = x[2i+1]*cos[i] + x[2i]*sin[i]
// elements at or beyond `rot` are copied.  q is rotated in place.
// Rotated k and v go to the pages: page = block_table[seq_of_token[n], p / block_size];
// a negative page (padding, or a page already given back) or p outside the table skips the write.
// K pages are [num_blocks, KV, block_size, d]; V pages are transposed, [num_blocks, KV, d,
// block_size], so that the keys of one element lie side by side (what the P*V product of the
// matrix cores contracts over).  With write_kv == 0 only q is rotated.
struct RopeArgs {
  int H, KV, d, rot, table_len, block_size, table_stride, num_blocks, write_kv, n_seqs;
};

template <typename T>
__global__ void rope_kvwrite_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                                    const int* __restrict__ seq_of_token,
                                    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                    const int* __restrict__ block_table, T* __restrict__ k_pages,
                                    T* __restrict__ v_pages, RopeArgs a) {
  const int n = blockIdx.x;
  const int p = positions[n];
  const int half = a.rot / 2;
  T* row = qkv + static_cast<size_t>(n) * (a.H + 2 * a.KV) * a.d;
  const bool pos_ok = p >= 0 && p < a.table_len;
  const float* cs = cos_t + static_cast<size_t>(pos_ok ? p : 0) * half;
  const float* sn = sin_t + static_cast<size_t>(pos_ok ? p : 0) * half;

  int page = -1, off = 0;
  if (a.write_kv && pos_ok) {
    const int seq = seq_of_token[n];
    const int blk = p / a.block_size;
    if (seq >= 0 && seq < a.n_seqs && blk < a.table_stride) {
      page = block_table[static_cast<size_t>(seq) * a.table_stride + blk];
      if (page >= a.num_blocks) page = -1;
      off = p - blk * a.block_size;
    }
  }
  // q heads: rotate in place (pairs are owned by one thread, so no hazard)
  const int q_pairs = a.H * half;
  for (int t = threadIdx.x; t < q_pairs; t += blockDim.x) {
    const int hh = t / half, i = t - hh * half;
    T* x = row + hh * a.d;
    const float x1 = Elem<T>::load(x + 2 * i), x2 = Elem<T>::load(x + 2 * i + 1);
    const float c = pos_ok ? cs[i] : 1.f, s = pos_ok ? sn[i] : 0.f;
    Elem<T>::store(x + 2 * i, x1 * c - x2 * s);
    Elem<T>::store(x + 2 * i + 1, x2 * c + x1 * s);
  }
  if (page < 0) return;
  // k heads: rotate, write to the page; the unrotated tail is copied
  const int k_pairs = a.KV * half;
  for (int t = threadIdx.x; t < k_pairs; t += blockDim.x) {
    const int hh = t / half, i = t - hh * half;
    const T* x = row + (a.H + hh) * a.d;
    T* dst = k_pages + ((static_cast<size_t>(page) * a.KV + hh) * a.block_size + off) * a.d;
    const float x1 = Elem<T>::load(x + 2 * i), x2 = Elem<T>::load(x + 2 * i + 1);
    Elem<T>::store(dst + 2 * i, x1 * cs[i] - x2 * sn[i]);
    Elem<T>::store(dst + 2 * i + 1, x2 * cs[i] + x1 * sn[i]);
  }
  const int tail = a.d - a.rot;
  for (int t = threadIdx.x; t < a.KV * tail; t += blockDim.x) {
    const int hh = t / tail, i = a.rot + (t - hh * tail);
    T* dst = k_pages + ((static_cast<size_t>(page) * a.KV + hh) * a.block_size + off) * a.d;
    dst[i] = row[(a.H + hh) * a.d + i];
  }
  for (int t = threadIdx.x; t < a.KV * a.d; t += blockDim.x) {
    const int hh = t / a.d, i = t - hh * a.d;
    v_pages[((static_cast<size_t>(page) * a.KV + hh) * a.d + i) * a.block_size + off] =
        row[(a.H + a.KV + hh) * a.d + i];
  }
}

// The same work for a tile of 16 tokens per workgroup with 8 elements per lane and access
// (d and the rotary width multiples of 8).  V is stored transposed, so a token's elements lie
// block_size apart; where the tile's 16 tokens fill consecutive places of one page (a prompt
// read from a page boundary) the tile is turned in LDS and each (head, element) row of 16
// tokens is stored in one piece.  Other tiles store V element by element.
constexpr int ROPE_TILE = 16;

__device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = static_cast<uint32_t>(f32_to_bf16(v[2 * i])) | (static_cast<uint32_t>(f32_to_bf16(v[2 * i + 1])) << 16);
  *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename T>
__global__ __launch_bounds__(256) void rope_kvwrite_tile_kernel(
    T* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ block_table, T* __restrict__ k_pages, T* __restrict__ v_pages, int n,
    int turn_v, RopeArgs a) {
  extern __shared__ __align__(16) unsigned char tile_raw[];  // [ROPE_TILE][V columns of this share] of T, if turn_v
  __shared__ int s_pos[ROPE_TILE], s_page[ROPE_TILE], s_off[ROPE_TILE], s_run;
  const int n0 = blockIdx.x * ROPE_TILE;
  const int cnt = min(ROPE_TILE, n - n0);
  const int half = a.rot / 2;
  if (threadIdx.x < ROPE_TILE) {
    const int t = threadIdx.x;
    int p = -1, page = -1, off = 0;
    if (t < cnt) {
      p = positions[n0 + t];
      if (p < 0 || p >= a.table_len) p = -1;
      if (p >= 0 && a.write_kv) {
        const int seq = seq_of_token[n0 + t];
        const int blk = p / a.block_size;
        if (seq >= 0 && seq < a.n_seqs && blk < a.table_stride) {
          page = block_table[static_cast<size_t>(seq) * a.table_stride + blk];
          if (page >= a.num_blocks) page = -1;
          off = p - blk * a.block_size;
        }
      }
    }
    s_pos[t] = p;
    s_page[t] = page;
    s_off[t] = off;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    bool run = turn_v && cnt == ROPE_TILE && s_page[0] >= 0 && s_off[0] % 8 == 0 &&
               a.block_size % 8 == 0 && s_off[0] + ROPE_TILE <= a.block_size;
    for (int t = 1; t < ROPE_TILE; ++t) run = run && s_page[t] == s_page[0] && s_off[t] == s_off[0] + t;
    s_run = run;
  }
  __syncthreads();
  // blockIdx.y names a share of the row: of its q and k vectors, and of its V columns
  const int row_len = (a.H + 2 * a.KV) * a.d;
  const int qk_vecs = (a.H + a.KV) * a.d / 8;
  const int qk_share = (qk_vecs + gridDim.y - 1) / gridDim.y;
  const int qk_begin = blockIdx.y * qk_share;
  const int qk_mine = max(0, min(qk_share, qk_vecs - qk_begin));
  for (int item = threadIdx.x; item < cnt * qk_mine; item += blockDim.x) {
    const int t = item / qk_mine, e = (qk_begin + item - t * qk_mine) * 8;
    const int head = e / a.d, i0 = e - head * a.d;
    const bool is_k = head >= a.H;
    const int p = s_pos[t], page = s_page[t];
    // a query that is not rotated stays as it is; a key without a page is not stored
    if (is_k ? page < 0 : (p < 0 || i0 >= a.rot)) continue;
    T* src = qkv + static_cast<size_t>(n0 + t) * row_len + e;
    float x[8];
    load8(src, x);
    if (p >= 0 && i0 < a.rot) {
      const float4 c = *reinterpret_cast<const float4*>(cos_t + static_cast<size_t>(p) * half + i0 / 2);
      const float4 sn = *reinterpret_cast<const float4*>(sin_t + static_cast<size_t>(p) * half + i0 / 2);
      const float cs[4] = {c.x, c.y, c.z, c.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float x1 = x[2 * i], x2 = x[2 * i + 1];
        x[2 * i] = x1 * cs[i] - x2 * ss[i];
        x[2 * i + 1] = x2 * cs[i] + x1 * ss[i];
      }
    }
    T* dst = is_k ? k_pages + ((static_cast<size_t>(page) * a.KV + (head - a.H)) * a.block_size + s_off[t]) * a.d + i0
                  : src;
    store8(dst, x);
  }
  if (!a.write_kv) return;
  const int v0 = (a.H + a.KV) * a.d, v_len = a.KV * a.d;
  const int v_share = (v_len / 8 + gridDim.y - 1) / gridDim.y * 8;  // columns, whole vectors
  const int v_begin = blockIdx.y * v_share;
  const int v_mine = max(0, min(v_share, v_len - v_begin));
  if (s_run) {
    T* tile = reinterpret_cast<T*>(tile_raw);  // [ROPE_TILE][v_share]
    const int v_vecs = v_mine / 8;
    for (int item = threadIdx.x; item < ROPE_TILE * v_vecs; item += blockDim.x) {
      const int t = item / v_vecs, e = (item - t * v_vecs) * 8;
      const T* src = qkv + static_cast<size_t>(n0 + t) * row_len + v0 + v_begin + e;
      constexpr int Q = sizeof(T) * 8 / 16;  // 16-byte pieces of eight elements
#pragma unroll
      for (int q = 0; q < Q; ++q)
        reinterpret_cast<uint4*>(tile + t * v_share + e)[q] = reinterpret_cast<const uint4*>(src)[q];
    }
    __syncthreads();
    const int page = s_page[0], off0 = s_off[0];
    for (int c = threadIdx.x; c < v_mine; c += blockDim.x) {  // v_begin + c = head * d + element
      __align__(16) T vals[ROPE_TILE];
#pragma unroll
      for (int t = 0; t < ROPE_TILE; ++t) vals[t] = tile[t * v_share + c];
      T* dst = v_pages + (static_cast<size_t>(page) * v_len + v_begin + c) * a.block_size + off0;
      constexpr int Q = sizeof(T) * ROPE_TILE / 16;
#pragma unroll
      for (int q = 0; q < Q; ++q) reinterpret_cast<uint4*>(dst)[q] = reinterpret_cast<const uint4*>(vals)[q];
    }
  } else {
    for (int item = threadIdx.x; item < cnt * v_mine; item += blockDim.x) {
      const int t = item / v_mine, c = v_begin + item - t * v_mine;
      const int page = s_page[t];
      if (page < 0) continue;
      v_pages[(static_cast<size_t>(page) * v_len + c) * a.block_size + s_off[t]] =
          qkv[static_cast<size_t>(n0 + t) * row_len + v0 + c];
    }
  }
}

template <typename T>
static int rope_launch(void* qkv, const int* positions, const int* seq_of_token, const float* cos_t,
                       const float* sin_t, const int* block_table, void* k_pages, void* v_pages,
                       int n, RopeArgs a, hipStream_t s) {
  if (n <= 0) return 0;
  if (a.d % 8 == 0 && a.rot % 8 == 0) {
    // few tiles: several workgroups share a tile's row, so that the chip has work
    const int tiles = (n + ROPE_TILE - 1) / ROPE_TILE;
    int shares = tiles >= 512 ? 1 : (512 + tiles - 1) / tiles;
    if (shares > 8) shares = 8;
    const int v_share = (a.KV * a.d / 8 + shares - 1) / shares * 8;
    // the tile of V rows turned in LDS; without room for it V goes element by element
    const size_t lds = static_cast<size_t>(ROPE_TILE) * v_share * sizeof(T);
    const int turn_v = lds <= 48 * 1024;
    hipLaunchKernelGGL(rope_kvwrite_tile_kernel<T>, dim3(tiles, shares), dim3(256), turn_v ? lds : 0, s,
                       static_cast<T*>(qkv), positions, seq_of_token, cos_t, sin_t, block_table,
                       static_cast<T*>(k_pages), static_cast<T*>(v_pages), n, turn_v, a);
    return kvf_last_error();
  }
  hipLaunchKernelGGL(rope_kvwrite_kernel<T>, dim3(n), dim3(128), 0, s, static_cast<T*>(qkv),
                     positions, seq_of_token, cos_t, sin_t, block_table, static_cast<T*>(k_pages),
                     static_cast<T*>(v_pages), a);
  return kvf_last_error();
}
#define ROPE_ARGS_DECL                                                                           \
  void *qkv, const int *positions, const int *seq_of_token, const float *cos_t,                 \
      const float *sin_t, const int *block_table, void *k_pages, void *v_pages, int n, int H,   \
      int KV, int d, int rot, int table_len, int block_size, int table_stride, int num_blocks,  \
      int write_kv, int n_seqs, hipStream_t s
#define ROPE_ARGS_PACK                                                                           \
  RopeArgs { H, KV, d, rot, table_len, block_size, table_stride, num_blocks, write_kv, n_seqs }
KVF_EXPORT int kvf_rope_kvwrite_f32(ROPE_ARGS_DECL) {
  return rope_launch<float>(qkv, positions, seq_of_token, cos_t, sin_t, block_table, k_pages,
                            v_pages, n, ROPE_ARGS_PACK, s);
}
KVF_EXPORT int kvf_rope_kvwrite_bf16(ROPE_ARGS_DECL) {
  return rope_launch<bf16_t>(qkv, positions, seq_of_token, cos_t, sin_t, block_table, k_pages,
                             v_pages, n, ROPE_ARGS_PACK, s);
}
