// C[M, N] = A[M, K] * W[N, K]^T for bf16 weights on the matrix cores (fp32 accumulation),
// built for few rows of A: the weight matrix is streamed once per pass of up to 16*MT rows and
// the kernel is bound by HBM, so all of the chip has to pull on W at once.
//
// One workgroup owns 16 rows of W (16 output columns).  Its waves split K: wave w takes the
// 32-wide k-steps w, w + nw, w + 2nw, ... so neighbouring waves read neighbouring 64-byte pieces
// of the same rows.  Per k-step a lane loads 16 B of W (row lane%16, k-offset 8*(lane/16)) and
// the matching 8 elements of each 16-row tile of A and issues one v_mfma_f32_16x16x32_bf16 per
// tile with W as the first operand, so a lane ends up holding four consecutive output columns of
// one row of C.  Partial sums of the waves are added in wave order through LDS.  With several
// row tiles of A (more than 16 rows) a wave takes NT neighbouring 16-row groups of W per k-step
// and reuses its A fragments for them, which divides the traffic for A (served by L2) by NT.
// The launch shape depends on N, K and on how many 16-row tiles a pass holds (1, 2, 4 or 8),
// never on the rows themselves.
//
// Left operand (AT): 0 = bf16 activations; 1 = the fp32 residual stream with the RMS norm folded
// in: y = x * rsqrt(mean(x^2) + eps) is applied as a per-row factor on the accumulators (the
// norm's weight vector is folded into W's columns when the model is loaded); the sum of squares
// is taken in fp32 from the same loads that feed the matrix cores.
//
// Epilogues (EPI): 0 store fp32; 1 store bf16; 2 add into fp32 (the residual stream);
// 3 SwiGLU gate: columns come in (gate, up) pairs, out[m, j] = silu(c[2j]) * c[2j+1] as bf16;
// 4 rotary + cache write for a fused q/k/v projection: neighbouring columns of q and k heads are
//   rotary pairs; rotated q goes to the output (bf16, q heads only), rotated k and plain v go
//   straight into the pages of the token's sequence (K pages [nb, KV, block, d], V pages
//   transposed [nb, KV, d, block]).
// 5 greedy pick for the output head of a decode step (at most 16 bf16 rows, already normalised:
//   with the norm folded in, each of the head's thousands of workgroups would read the fp32 rows
//   and their sums of squares again, as many bytes as the matrix itself): no logits are stored;
//   every workgroup leaves the best (value, column) of its columns per row in a workspace and
//   takes a ticket, and the workgroup that takes the last one picks every row's best over all
//   workgroups (the lowest column among equal values), then does what the step's tail would
//   need kernels of their own for: it hands the tokens out, makes each sequence's token its
//   next input (token id, position and context length move on by one), keeps the tokens in the
//   ring row of this step for the host, and writes the tokens' embedding rows into the residual
//   stream for the next step.
// K must be a multiple of 8 (16-byte loads); a k-step that passes K loads zeros.
//
// A product that is added to a narrow C over a long K (the down projection) has fewer workgroups
// than the chip has compute units, and a compute unit keeps only so many bytes in flight.  It
// may be cut into two halves of K (`Riders::half_out`): a second layer of workgroups stores its
// half beside C (rounded to bf16, as a product that is stored is), and the caller owes that half
// to C.  The next consumers add it on their way:
// the fused q/k/v projection in its loads (`a_add`), the output projection in its sum (`c_add`).
//
// Layout of W.  In the checkpoint's row-major [N, K] a wave's load of one operand fragment
// touches 16 rows, 64 bytes each: 16 cache lines per group of 16 lanes, and the L1 looks lines up
// one at a time, which bounds the kernel far below what HBM delivers.  The engine therefore also
// keeps W in tiles (`w_tiled`): [ceil(N/16)][ceil(K/32)][64 lanes][8 elements], tile (g, s) being
// rows 16g..16g+15, columns 32s..32s+31 in the order the instruction wants them (lane
// 16*c + r holds row r, columns 8c..8c+7), zero-padded.  A fragment is then 1 KB of consecutive
// bytes.  Both layouts give the same bits.
#include "common.h"

namespace {
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

struct RopeEpi {
  const int* positions;
  const int* seq_of_token;
  const float* cos_t;
  const float* sin_t;
  const int* block_table;
  bf16_t* k_pages;
  bf16_t* v_pages;
  int H, KV, d, rot, table_len, block_size, table_stride, num_blocks, write_kv, n_seqs;
};

// Sums that ride along, all bf16 (a workgroup of the fused projection reads every row of A and
// of a_add: with the addend in fp32 that was as many bytes again as A, 1.8 us of a 8.6 us kernel
// at eight rows).  `a_add` (kernels built with ADD): the left operand is A + a_add, A in fp32,
// the same row stride counted in elements.  `c_add` (with EPI 2): C += product + c_add, row
// stride of C.
// `half_out` (with EPI 2): the grid is two deep; workgroups of the second layer walk the second
// half of K and store their product there (fp32, row stride of C) instead of adding it to C, so
// that a narrow C still puts a workgroup on every compute unit; the caller owes half_out to C.
struct Riders {
  const bf16_t* a_add;
  const bf16_t* c_add;
  bf16_t* half_out;
};

// Operands of the greedy pick (EPI 5).  part_val / part_idx: [16][workgroups] and behind them
// [16][PICK_LANES] scratch; ticket:
// PICK_TICKET_INTS ints, zero between launches (atomics on one address are served one after the
// other, some 65 ns each on this chip, and thousands of workgroups on one counter would queue
// for longer than the product takes: the workgroups are spread over PICK_LANES counters, a
// cache line apart, and the last arrival at each takes a ticket of a second counter).  tokens: [M] out.  token_ids / positions / ctx_lens: the step's
// inputs, advanced in place; ring [ring_rows][ring_stride] and run_counter as decode_advance
// takes them.  embed [vocab][hidden] bf16 -> residual [M][ld_res] fp32 for the next step.
struct PickEpi {
  float* part_val;
  int* part_idx;
  int* ticket;
  int* tokens;
  int* token_ids;
  int* positions;
  int* ctx_lens;
  int* ring;
  int* run_counter;
  const bf16_t* embed;
  float* residual;
  int ring_stride, ring_rows, hidden, ld_res;
};

constexpr int PICK_LANES = 64, PICK_STRIDE = 16;   // counters, and ints between two of them
constexpr int PICK_TICKET_INTS = (PICK_LANES + 1) * PICK_STRIDE;

// True in the caller (one thread asks) that arrives last of `expected` at `counter`, which it
// leaves zero.  Every caller has made its results visible before.
__device__ __forceinline__ bool pick_last_at(int* counter, int expected) {
  if (atomicAdd(counter, 1) != expected - 1) return false;
  __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
  return v > bv || (v == bv && i < bi);
}

// Results that other workgroups are going to read are stored past this XCD's L2 (an atomic store
// at device scope is written through); before a ticket is taken they have to be complete.
// A device-scope release fence would also write the whole L2's dirty lines back, and thousands
// of workgroups doing that made the head's product take 275 us instead of 90.  What orders the
// results before the ticket instead: every wave that published waits until its stores have been
// acknowledged (the vector memory counter at zero: a written-through store is acknowledged from
// where the device's other L2s read it), then comes the workgroup's barrier, and only then does
// thread 0 add to the ticket.  A fence of workgroup scope alone would not do: it lets stores to
// global memory stay in flight, since all waves of a workgroup share one L1.
__device__ __forceinline__ void pick_publish(float* val, int* idx, size_t at, float v, int i) {
  __hip_atomic_store(val + at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(idx + at, i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void pick_stores_done() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// The last arrival at counter `lane`: the best per row over the workgroups lane, lane + 64, ...
// into the second level of the scratch ([16][PICK_LANES] behind the first).  All threads of the
// workgroup; plain loads after the caller's acquire fence.
__device__ __forceinline__ void pick_merge_lane(const PickEpi& pk, int M, int groups, int lane) {
  const int tid = threadIdx.x, sub = tid % 32;    // 32 threads per row, rows in turn
  for (int row = tid / 32; row < 16; row += blockDim.x / 32) {   // the same trips in every thread
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    if (row < M) {
      for (int c = lane + sub * PICK_LANES; c < groups; c += 32 * PICK_LANES) {
        const float v = pk.part_val[row * groups + c];
        const int i = pk.part_idx[row * groups + c];
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
      }
    }
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, KVF_WAVE);
      const int oi = __shfl_xor(bi, o, KVF_WAVE);
      if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if (sub == 0 && row < M)
      pick_publish(pk.part_val + 16 * groups, pk.part_idx + 16 * groups, row * PICK_LANES + lane, bv, bi);
  }
  pick_stores_done();
}

// The last workgroup of a greedy pick: see EPI 5 at the head of the file.  `lds` holds at least
// 16 ints.
__device__ __forceinline__ void pick_finish(const PickEpi& pk, int M, int groups, float* lds) {
  const int tid = threadIdx.x;
  const int lanes = groups < PICK_LANES ? groups : PICK_LANES;
  int* tok = reinterpret_cast<int*>(lds);   // [16]
  // 16 threads per row over the second level's (at most 64) candidates, rows in turn
  for (int row = tid / 16; row < 16; row += blockDim.x / 16) {
    const int sub = tid % 16;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    if (row < M) {
      for (int c = sub; c < lanes; c += 16) {
        const float v = pk.part_val[16 * groups + row * PICK_LANES + c];
        const int i = pk.part_idx[16 * groups + row * PICK_LANES + c];
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
      }
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, KVF_WAVE);
      const int oi = __shfl_xor(bi, o, KVF_WAVE);
      if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if (sub == 0 && row < M) tok[row] = bi == 0x7fffffff ? 0 : bi;
  }
  const int step = *pk.run_counter;   // read by every thread before it moves
  __syncthreads();
  if (tid < M) {
    const int t = tok[tid];
    pk.tokens[tid] = t;
    if (step >= 0 && step < pk.ring_rows) pk.ring[step * pk.ring_stride + tid] = t;
    if (pk.ctx_lens[tid] > 0) {     // padding sequences stay empty
      pk.token_ids[tid] = t;
      pk.positions[tid] += 1;
      pk.ctx_lens[tid] += 1;
    }
  }
  if (tid == 0) *pk.run_counter = step + 1;
  __syncthreads();
  // the tokens' embedding rows, widened, are the next step's residual stream
  const int per_row = pk.hidden / 8;
  for (int idx = tid; idx < M * per_row; idx += blockDim.x) {
    const int r = idx / per_row, k = (idx - r * per_row) * 8;
    float v[8];
    load8(pk.embed + static_cast<size_t>(tok[r]) * pk.hidden + k, v);
    float* dst = pk.residual + static_cast<size_t>(r) * pk.ld_res + k;
    *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
}

__device__ __forceinline__ bf16x8 load_frag(const bf16_t* p, bool ok) {
  uint4 r = make_uint4(0u, 0u, 0u, 0u);
  if (ok) r = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, r);
}

// 8 fp32 (with ADD plus 8 of `q`) -> 8 bf16 (round to nearest even); adds their squares to ss.
// Nothing inside the branches uses what they load, so no branch ends in a wait and the loads of
// a whole pass stay in flight together.
template <bool ADD>
__device__ __forceinline__ bf16x8 load_frag_f32(const float* p, const bf16_t* q, bool ok, float& ss) {
  typedef __attribute__((ext_vector_type(8))) float f32x8;
  float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  uint4 raw = make_uint4(0u, 0u, 0u, 0u);   // eight bf16 of q, widened after the branch
  if (ok) {
    load8(p, v);
    if (ADD) raw = *reinterpret_cast<const uint4*>(q);
  }
  const float w[8] = {__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                      __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u),
                      __uint_as_float(raw.z << 16), __uint_as_float(raw.z & 0xffff0000u),
                      __uint_as_float(raw.w << 16), __uint_as_float(raw.w & 0xffff0000u)};
  f32x8 x;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float t = ADD ? v[i] + w[i] : v[i];
    ss = fmaf(t, t, ss);
    x[i] = t;
  }
  return __builtin_convertvector(x, bf16x8);
}

// What an epilogue reads besides the accumulators.  With one row tile the lanes of wave 0 finish
// the workgroup's tile and know their row and columns from the start, so they ask for these
// operands before the walk over K and find them in registers afterwards, instead of paying
// their latencies (up to three dependent loads for the cache write) at the end.
struct EpiOperands {
  f32x4 c;            // EPI 2: the four values the product is added to
  int pos, page;      // EPI 4: the token's position; the page its key and value go to (or -1)
  float cs[2], sn[2]; // EPI 4: rotation of the lane's two pairs
  bool have;
};

// 16-byte accesses to C are possible where rows and base are aligned and all four columns exist
__device__ __forceinline__ bool vec4_ok(const void* Cv, int ldc, int n, int N, int elem) {
  return n + 3 < N && (ldc * elem) % 16 == 0 && n % 4 == 0 &&
         reinterpret_cast<uintptr_t>(Cv) % 16 == 0;
}

// First stage: loads that need only (m, n).
template <int EPI>
__device__ __forceinline__ void epi_prefetch_a(EpiOperands& op, int m, int n, int N, int ldc, const void* Cv,
                                               const bf16_t* c_add, const RopeEpi& rp) {
  op.have = true;
  if (EPI == 2) {
    const size_t idx = static_cast<size_t>(m) * ldc + n;
    const float* c = static_cast<const float*>(Cv) + idx;
    if (vec4_ok(Cv, ldc, n, N, 4) && vec4_ok(c_add, ldc, n, N, 2)) {
      op.c = *reinterpret_cast<const f32x4*>(c);
      if (c_add) {
        const uint2 packed = *reinterpret_cast<const uint2*>(c_add + idx);
        op.c += f32x4{__uint_as_float(packed.x << 16), __uint_as_float(packed.x & 0xffff0000u),
                      __uint_as_float(packed.y << 16), __uint_as_float(packed.y & 0xffff0000u)};
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        op.c[r] = n + r < N ? c[r] + (c_add ? bf16_to_f32(c_add[idx + r].bits) : 0.f) : 0.f;
    }
  }
  if (EPI == 4) {
    op.pos = rp.positions[m];
    op.page = rp.write_kv ? rp.seq_of_token[m] : -1;  // the sequence for now
  }
}
// Second stage: loads that need what the first brought (position -> angles, sequence -> page).
template <int EPI>
__device__ __forceinline__ void epi_prefetch_b(EpiOperands& op, int n, const RopeEpi& rp) {
  if (EPI != 4) return;
  const int head = n / rp.d, e = n - head * rp.d;
  const int p = op.pos;
  const bool pos_ok = p >= 0 && p < rp.table_len;
#pragma unroll
  for (int pr = 0; pr < 2; ++pr) {
    const int j = (e + 2 * pr) / 2;
    const bool rotate = head < rp.H + rp.KV && pos_ok && 2 * j + 1 < rp.rot;
    op.cs[pr] = rotate ? rp.cos_t[static_cast<size_t>(p) * (rp.rot / 2) + j] : 1.f;
    op.sn[pr] = rotate ? rp.sin_t[static_cast<size_t>(p) * (rp.rot / 2) + j] : 0.f;
  }
  const int seq = op.page;
  int page = -1;
  if (head >= rp.H && rp.write_kv && pos_ok) {
    const int blk = p / rp.block_size;
    if (seq >= 0 && seq < rp.n_seqs && blk < rp.table_stride)
      page = rp.block_table[static_cast<size_t>(seq) * rp.table_stride + blk];
  }
  op.page = page;
}

// One lane's four neighbouring columns n..n+3 of row m, after the waves' partial sums are added.
template <int EPI>
__device__ __forceinline__ void store_tile(const f32x4& s, int m, int n, int N, int ldc, void* Cv,
                                           const bf16_t* c_add, const RopeEpi& rp, EpiOperands& op) {
  if (EPI == 2 || EPI == 4) {
    if (!op.have) {
      epi_prefetch_a<EPI>(op, m, n, N, ldc, Cv, c_add, rp);
      epi_prefetch_b<EPI>(op, n, rp);
    }
  }
  if (EPI <= 2) {
    const size_t idx = static_cast<size_t>(m) * ldc + n;
    if (EPI == 0 && vec4_ok(Cv, ldc, n, N, 4)) {
      *reinterpret_cast<f32x4*>(static_cast<float*>(Cv) + idx) = s;
    } else if (EPI == 2 && vec4_ok(Cv, ldc, n, N, 4)) {
      *reinterpret_cast<f32x4*>(static_cast<float*>(Cv) + idx) = op.c + s;
    } else if (EPI == 1 && vec4_ok(Cv, ldc, n, N, 2)) {
      uint2 packed;
      packed.x = static_cast<uint32_t>(f32_to_bf16(s[0])) | (static_cast<uint32_t>(f32_to_bf16(s[1])) << 16);
      packed.y = static_cast<uint32_t>(f32_to_bf16(s[2])) | (static_cast<uint32_t>(f32_to_bf16(s[3])) << 16);
      *reinterpret_cast<uint2*>(static_cast<bf16_t*>(Cv) + idx) = packed;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (n + r >= N) break;
        if (EPI == 0) static_cast<float*>(Cv)[idx + r] = s[r];
        if (EPI == 1) static_cast<bf16_t*>(Cv)[idx + r].bits = f32_to_bf16(s[r]);
        if (EPI == 2) static_cast<float*>(Cv)[idx + r] = op.c[r] + s[r];
      }
    }
  } else if (EPI == 3) {
    // N is even and n a multiple of 4: two (gate, up) pairs
    bf16_t* o = static_cast<bf16_t*>(Cv) + static_cast<size_t>(m) * ldc + n / 2;
    o[0].bits = f32_to_bf16(s[0] / (1.f + __expf(-s[0])) * s[1]);
    if (n + 2 < N) o[1].bits = f32_to_bf16(s[2] / (1.f + __expf(-s[2])) * s[3]);
  } else {
    // fused q/k/v projection: d is a multiple of 4, so the four columns lie in one head; pairs
    // that are not rotated (v heads, elements past the rotary width, positions off the table)
    // carry the identity
    const int head = n / rp.d, e = n - head * rp.d;
    float o[4];
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      const float x1 = s[2 * pr], x2 = s[2 * pr + 1];
      o[2 * pr] = x1 * op.cs[pr] - x2 * op.sn[pr];
      o[2 * pr + 1] = x2 * op.cs[pr] + x1 * op.sn[pr];
    }
    uint2 packed;
    packed.x = static_cast<uint32_t>(f32_to_bf16(o[0])) | (static_cast<uint32_t>(f32_to_bf16(o[1])) << 16);
    packed.y = static_cast<uint32_t>(f32_to_bf16(o[2])) | (static_cast<uint32_t>(f32_to_bf16(o[3])) << 16);
    if (head < rp.H) {
      *reinterpret_cast<uint2*>(static_cast<bf16_t*>(Cv) + static_cast<size_t>(m) * ldc + n) = packed;
    } else if (op.page >= 0 && op.page < rp.num_blocks) {
      const int off = op.pos % rp.block_size;
      if (head < rp.H + rp.KV) {
        const int kvh = head - rp.H;
        *reinterpret_cast<uint2*>(
            rp.k_pages + ((static_cast<size_t>(op.page) * rp.KV + kvh) * rp.block_size + off) * rp.d + e) =
            packed;
      } else {
        // V pages are [num_blocks, KV, d, block_size]: one element per key row
        const int kvh = head - rp.H - rp.KV;
        bf16_t* dst =
            rp.v_pages + ((static_cast<size_t>(op.page) * rp.KV + kvh) * rp.d + e) * rp.block_size + off;
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[static_cast<size_t>(r) * rp.block_size].bits = f32_to_bf16(o[r]);
      }
    }
  }
}

// more tiles per wave mean more registers per lane and more LDS per wave: fewer waves; fp32
// rows take twice the registers while in flight
constexpr int max_waves(int mt, int nt, int at) {
  return (mt * nt >= 8 || (at && mt >= 4)) ? 4 : (mt * nt >= 4 || (at && mt >= 2)) ? 8 : 16;
}
// k-steps whose loads are in flight together in one wave
constexpr int depth(int mt, int nt, int at) {
  return at ? (mt == 1 ? 4 : mt <= 4 ? 2 : 1) : (mt * nt == 1 ? 8 : mt * nt <= 4 ? 4 : 2);
}

template <int MT, int NT, int AT, int EPI, bool ADD>
__global__ __launch_bounds__(max_waves(MT, NT, AT) * KVF_WAVE) void gemm_skinny_kernel(
    const void* __restrict__ Av, const bf16_t* __restrict__ W, void* __restrict__ Cv, int M, int N,
    int K, int lda, int ldc, int m_base, float eps, int w_tiled, Riders rd, RopeEpi rp, PickEpi pk) {
  constexpr int RW = 16;  // rows of W per group
  extern __shared__ float red[];  // [nw][MT][64 lanes][4], then [nw][MT][16] sums of squares
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int nw = blockDim.x / KVF_WAVE;
  const int n0 = blockIdx.x * RW * NT;
  const int r16 = lane % 16, kg = lane / 16;
  const int ksteps = (K + 31) / 32;
  // the k-steps this workgroup walks: all, or one half of them (see Riders::half_out)
  const bool halves = EPI == 2 && rd.half_out != nullptr;
  const bool second = halves && blockIdx.y == 1;
  const int ks_cut = halves ? (ksteps + 1) / 2 : ksteps;
  const int ks_lo = second ? ks_cut : 0, ks_hi = second ? ksteps : ks_cut;
  // where this lane's fragment of k-step 0 lies, and how far the next k-step is
  const bf16_t* wp[NT];
  const size_t w_step = w_tiled ? KVF_WAVE * 8 : 32;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (w_tiled) {
      const int group = min(static_cast<int>(blockIdx.x) * NT + j, (N + RW - 1) / RW - 1);
      wp[j] = W + (static_cast<size_t>(group) * ksteps * KVF_WAVE + lane) * 8;
    } else {
      int wrow = n0 + j * RW + r16;
      if (wrow >= N) wrow = N - 1;  // clamped rows are computed and never stored
      wp[j] = W + static_cast<size_t>(wrow) * K + kg * 8;
    }
  }
  size_t aoff[MT];
  bool a_live[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    // Rows past M are not loaded at all (their lanes hold zeros and are never stored): a wave's
    // load touches one cache line per row it reads, and the L1 looks lines up one at a time.
    const int arow = m_base + t * 16 + r16;
    a_live[t] = arow < M;
    aoff[t] = static_cast<size_t>(a_live[t] ? arow : 0) * lda + kg * 8;
  }
  const bf16_t* Ab = static_cast<const bf16_t*>(Av);
  const float* Af = static_cast<const float*>(Av);
  const bf16_t* a_add = ADD ? rd.a_add : nullptr;
  const bf16_t* c_add = EPI == 2 && !second ? rd.c_add : nullptr;
  f32x4 acc[NT][MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    ss[t] = 0.f;
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // With one row tile, lane l of wave 0 will finish C[m_base + l%16][n0 + j*RW + 4*(l/16) ..+3]:
  // it asks for what its epilogue reads now, and for what depends on that after its first pass.
  constexpr bool PRE = MT == 1 && (EPI == 2 || EPI == 4);
  EpiOperands pre[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) pre[j].have = false;
  const int pre_m = m_base + r16, pre_n = n0 + 4 * kg;
  const bool pre_mine = PRE && wave == 0 && pre_m < M && !second;
  if (pre_mine) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
      if (pre_n + j * RW < N) epi_prefetch_a<EPI>(pre[j], pre_m, pre_n + j * RW, N, ldc, Cv, c_add, rp);
  }

  constexpr int U = depth(MT, NT, AT);
  int ks = ks_lo + wave;
  bool first = true;
  for (; ks + (U - 1) * nw < ks_hi; ks += U * nw) {
    bf16x8 wf[U][NT], af[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (ks + u * nw) * 32;
      const bool ok = k + kg * 8 + 8 <= K;
#pragma unroll
      for (int j = 0; j < NT; ++j) wf[u][j] = load_frag(wp[j] + (ks + u * nw) * w_step, ok || w_tiled);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        af[u][t] = AT ? load_frag_f32<ADD>(Af + aoff[t] + k, a_add + aoff[t] + k, ok && a_live[t], ss[t])
                      : load_frag(Ab + aoff[t] + k, ok && a_live[t]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][j], af[u][t], acc[j][t], 0, 0, 0);
    if (PRE && first) {  // the first stage has arrived with this pass's loads
      first = false;
      if (pre_mine) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
          if (pre[j].have) epi_prefetch_b<EPI>(pre[j], pre_n + j * RW, rp);
      }
    }
  }
  if (PRE && first && pre_mine) {  // K too short for a full pass
#pragma unroll
    for (int j = 0; j < NT; ++j)
      if (pre[j].have) epi_prefetch_b<EPI>(pre[j], pre_n + j * RW, rp);
  }
  for (; ks < ks_hi; ks += nw) {
    const int k = ks * 32;
    const bool ok = k + kg * 8 + 8 <= K;
    bf16x8 af[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
      af[t] = AT ? load_frag_f32<ADD>(Af + aoff[t] + k, a_add + aoff[t] + k, ok && a_live[t], ss[t])
                 : load_frag(Ab + aoff[t] + k, ok && a_live[t]);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const bf16x8 wf = load_frag(wp[j] + ks * w_step, ok || w_tiled);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af[t], acc[j][t], 0, 0, 0);
    }
  }
  // lane holds C[row r16][cols n0 + 16*j + 4*kg .. +3] of each tile
  float pick_v = -INFINITY;   // EPI 5: the best of this thread's columns of its row so far
  int pick_i = 0x7fffffff;
  float* red_ss = red + nw * MT * KVF_WAVE * 4;
  if (AT) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float v = ss[t];
      v += __shfl_xor(v, 16, KVF_WAVE);
      v += __shfl_xor(v, 32, KVF_WAVE);
      if (kg == 0) red_ss[(wave * MT + t) * 16 + r16] = v;
    }
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (j > 0) __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t)
      *reinterpret_cast<f32x4*>(red + ((wave * MT + t) * KVF_WAVE + lane) * 4) = acc[j][t];
    __syncthreads();
    for (int item = threadIdx.x; item < MT * KVF_WAVE; item += blockDim.x) {
      const int t = item / KVF_WAVE, l = item % KVF_WAVE;
      f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < nw; ++w)
        s += *reinterpret_cast<const f32x4*>(red + ((w * MT + t) * KVF_WAVE + l) * 4);
      const int m = m_base + t * 16 + l % 16;
      const int n = n0 + j * RW + 4 * (l / 16);
      if (m >= M || n >= N) continue;
      if (AT) {
        float tot = 0.f;
        for (int w = 0; w < nw; ++w) tot += red_ss[(w * MT + t) * 16 + l % 16];
        s *= rsqrtf(tot / static_cast<float>(K) + eps);
      }
      if (EPI == 5) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N && better(s[r], n + r, pick_v, pick_i)) { pick_v = s[r]; pick_i = n + r; }
        continue;
      }
      EpiOperands fresh;
      fresh.have = false;
      if (EPI == 2 && second)
        store_tile<1>(s, m, n, N, ldc, rd.half_out, nullptr, rp, fresh);
      else
        store_tile<EPI>(s, m, n, N, ldc, Cv, c_add, rp, PRE ? pre[j] : fresh);
    }
  }
  if (EPI == 5) {
    // one row tile: the first 64 threads hold row r16's best over their four columns of every
    // group of this workgroup
    if (wave == 0) {
#pragma unroll
      for (int o = 16; o <= 32; o <<= 1) {
        const float ov = __shfl_xor(pick_v, o, KVF_WAVE);
        const int oi = __shfl_xor(pick_i, o, KVF_WAVE);
        if (better(ov, oi, pick_v, pick_i)) { pick_v = ov; pick_i = oi; }
      }
      const int m = m_base + r16;
      if (kg == 0 && m < M)
        pick_publish(pk.part_val, pk.part_idx, static_cast<size_t>(m) * gridDim.x + blockIdx.x, pick_v, pick_i);
      pick_stores_done();
    }
    // Two levels of tickets: the workgroups are spread over PICK_LANES counters; the last
    // arrival at a counter merges that counter's workgroups and takes a ticket of the top
    // counter; the last arrival there finishes.
    const int groups = static_cast<int>(gridDim.x), lane_id = static_cast<int>(blockIdx.x) % PICK_LANES;
    int* flag = reinterpret_cast<int*>(red);
    __syncthreads();     // (and nobody reads `red` any more)
    if (threadIdx.x == 0)
      flag[0] = pick_last_at(pk.ticket + lane_id * PICK_STRIDE, (groups - lane_id + PICK_LANES - 1) / PICK_LANES);
    __syncthreads();
    if (flag[0] == 0) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // what the others published, not this XCD's stale copy
    pick_merge_lane(pk, M, groups, lane_id);
    __syncthreads();
    if (threadIdx.x == 0)
      flag[1] = pick_last_at(pk.ticket + PICK_LANES * PICK_STRIDE, groups < PICK_LANES ? groups : PICK_LANES);
    __syncthreads();
    if (flag[1] == 0) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    pick_finish(pk, M, groups, red + 64);
  }
}

int g_waves_override = 0;
int g_rows_override = 0;

// Waves per workgroup, as measured on the shapes of a 1B-parameter decoder: eight (fewer leave
// loads unhidden, sixteen crowd the CU); at least one k-step per wave.
int pick_waves(int K) {
  const int ksteps = (K + 31) / 32;
  int nw = g_waves_override > 0 ? g_waves_override : 8;
  if (nw > 16) nw = 16;
  if (nw > ksteps) nw = ksteps;
  if (nw < 1) nw = 1;
  return nw;
}

template <int MT, int NT, int AT, int EPI>
int launch_one(const void* A, const bf16_t* W, void* C, int M, int N, int K, int lda, int ldc,
               int m_base, float eps, int w_tiled, const Riders& rd, const RopeEpi& rp, hipStream_t s,
               const PickEpi& pk = PickEpi{}) {
  const int groups = (N + 16 * NT - 1) / (16 * NT);
  int nw = pick_waves(K);
  if (nw > max_waves(MT, NT, AT)) nw = max_waves(MT, NT, AT);
  const dim3 grid(groups, EPI == 2 && rd.half_out ? 2 : 1), block(nw * KVF_WAVE);
  size_t lds = static_cast<size_t>(nw) * MT * (KVF_WAVE * 4 + 16) * sizeof(float);
  if (EPI == 5 && lds < (64 + 2 * 16 * 16 + 16) * sizeof(float)) lds = (64 + 2 * 16 * 16 + 16) * sizeof(float);
  if (rd.a_add) {
    // the sum that rides in the left operand's loads: only the fused q/k/v projection of one
    // tile of rows is built with it
    if constexpr (MT == 1 && AT == 1 && EPI == 4)
      hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT, AT, EPI, true>), grid, block, lds, s, A, W, C, M, N, K,
                         lda, ldc, m_base, eps, w_tiled, rd, rp, pk);
    else
      return static_cast<int>(hipErrorInvalidValue);
  } else {
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT, AT, EPI, false>), grid, block, lds, s, A, W, C, M, N, K,
                       lda, ldc, m_base, eps, w_tiled, rd, rp, pk);
  }
  return kvf_last_error();
}

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

// How many 16-row groups of W a wave takes when A has several row tiles.  With 17 to 64 rows the
// product is bound by what every compute unit has to bring in through its L1, which keeps only
// some fifty lines in flight: all rows of A for each of its workgroups, and their columns of W.
// A wave that takes more groups shares A's rows among more columns, but leaves fewer
// workgroups; the choice is the one with the least to fill per compute unit, in rounds of
// workgroups over the chip (measured at 32 rows: [5120, 3072] 15.2 us with one group, 10.9 with
// two; [28672, 4096] 62.8 with two, 53.3 with four).
template <int MT, int AT, int EPI>
int launch_nt(const void* A, const bf16_t* W, void* C, int M, int N, int K, int lda, int ldc,
              int m_base, float eps, int w_tiled, const Riders& rd, const RopeEpi& rp, hipStream_t s) {
  const int tiles = (N + 15) / 16;
  if constexpr (MT >= 2 && MT <= 4 && !AT) {
    const int cus = compute_units(), rows = M - m_base < MT * 16 ? M - m_base : MT * 16;
    int best = 1, least = 0x7fffffff;
    for (int nt = 1; nt <= 4; nt *= 2) {
      const int groups = (tiles + nt - 1) / nt;
      const int fill = ((groups + cus - 1) / cus) * (rows + 16 * nt);
      if (fill < least) {
        least = fill;
        best = nt;
      }
    }
    if (best == 4)
      return launch_one<MT, 4, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
    if (best == 2)
      return launch_one<MT, 2, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
  }
  if (MT == 1) {
    // Every workgroup reads all of A, so with several rows of A and many rows of W a workgroup
    // takes 32 rows of W and halves that traffic; fp32 rows weigh twice as much and make it pay
    // with fewer rows of W.
    const int rw = g_rows_override > 0 ? g_rows_override : (M - m_base > 4 && tiles >= (AT ? 256 : 512) ? 32 : 16);
    if (rw == 32) return launch_one<1, 2, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
    if (rw == 64) return launch_one<1, 4, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
  }
  return launch_one<MT, 1, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
}

template <int AT, int EPI>
int launch_rows(const void* A, const bf16_t* W, void* C, int M, int N, int K, int lda, int ldc,
                float eps, int w_tiled, const Riders& rd, const RopeEpi& rp, hipStream_t s) {
  int err = 0;
  for (int m_base = 0; m_base < M && !err; m_base += 128) {
    const int rows = M - m_base < 128 ? M - m_base : 128;
    if (rows <= 16) err = launch_nt<1, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
    else if (rows <= 32) err = launch_nt<2, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
    else if (rows <= 64) err = launch_nt<4, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
    else err = launch_nt<8, AT, EPI>(A, W, C, M, N, K, lda, ldc, m_base, eps, w_tiled, rd, rp, s);
  }
  return err;
}

template <int AT>
int launch_epi(const void* A, const bf16_t* W, void* C, int epi, int M, int N, int K, int lda,
               int ldc, float eps, int w_tiled, const Riders& rd, const RopeEpi& rp, hipStream_t s) {
  switch (epi) {
    case 0: return launch_rows<AT, 0>(A, W, C, M, N, K, lda, ldc, eps, w_tiled, rd, rp, s);
    case 1: return launch_rows<AT, 1>(A, W, C, M, N, K, lda, ldc, eps, w_tiled, rd, rp, s);
    case 2: return launch_rows<AT, 2>(A, W, C, M, N, K, lda, ldc, eps, w_tiled, rd, rp, s);
    case 3: return launch_rows<AT, 3>(A, W, C, M, N, K, lda, ldc, eps, w_tiled, rd, rp, s);
    case 4: return launch_rows<AT, 4>(A, W, C, M, N, K, lda, ldc, eps, w_tiled, rd, rp, s);
  }
  return static_cast<int>(hipErrorInvalidValue);
}
}  // namespace

// For measurements: force the number of waves per workgroup and the rows of W per workgroup
// (0 = choose by shape).
KVF_EXPORT void kvf_gemm_bf16_set_waves(int waves) { g_waves_override = waves; }
KVF_EXPORT void kvf_gemm_bf16_set_rows(int rows) { g_rows_override = rows; }

// a_type: 0 = bf16 rows, 1 = fp32 rows normalised by rsqrt(mean(x^2) + eps) in the kernel.
// epi: 0 store fp32, 1 store bf16, 2 add into fp32, 3 SwiGLU pairs -> bf16 [M, N/2].
// w_tiled: W is [N, K] row-major (0) or in tiles of 16 x 32 (1, see the head of this file).
// c_add (epi 2 only, may be null): bf16 [M, ldc], added to C together with the product.
// half_out (epi 2 with bf16 rows only, may be null): bf16 [M, ldc]; the product over the second
//   half of K is stored there instead of being added to C, by a second layer of workgroups.
KVF_EXPORT int kvf_gemm_bf16(const void* A, int a_type, const void* W, int w_tiled, void* C, int epi,
                             int M, int N, int K, int lda, int ldc, float eps, const void* c_add,
                             void* half_out, hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8 != 0 || lda % 8 != 0 || epi < 0 || epi > 3 || (epi == 3 && N % 4 != 0))
    return static_cast<int>(hipErrorInvalidValue);
  if (((c_add || half_out) && epi != 2) || (half_out && (a_type != 0 || K < 64)))
    return static_cast<int>(hipErrorInvalidValue);
  const RopeEpi none{};
  const Riders rd{nullptr, static_cast<const bf16_t*>(c_add), static_cast<bf16_t*>(half_out)};
  const bf16_t* w = static_cast<const bf16_t*>(W);
  if (a_type == 0) return launch_epi<0>(A, w, C, epi, M, N, K, lda, ldc, eps, w_tiled, rd, none, s);
  if (a_type == 1) return launch_epi<1>(A, w, C, epi, M, N, K, lda, ldc, eps, w_tiled, rd, none, s);
  return static_cast<int>(hipErrorInvalidValue);
}

// Fused q/k/v projection with rotary and cache write.  W: [(H + 2*KV) * d, K] with q and k rows
// permuted so that rotary pairs are neighbouring rows.  q_out: [M, ldq >= H * d] bf16.
// a_add (a_type 1 and at most 16 rows only, may be null): bf16 [M, lda], added to A before the
// norm.
KVF_EXPORT int kvf_gemm_bf16_qkv_rope(const void* A, int a_type, const void* W, int w_tiled,
                                      void* q_out, int M, int K, int lda, int ldq, float eps,
                                      const void* a_add, const int* positions,
                                      const int* seq_of_token, const float* cos_t,
                                      const float* sin_t, const int* block_table, void* k_pages,
                                      void* v_pages, int H, int KV, int d, int rot, int table_len,
                                      int block_size, int table_stride, int num_blocks,
                                      int write_kv, int n_seqs, hipStream_t s) {
  if (M <= 0) return 0;
  if (K <= 0 || K % 8 != 0 || lda % 8 != 0 || d % 4 != 0 || rot % 2 != 0 || rot > d || ldq % 4 != 0 ||
      (a_add && (a_type != 1 || M > 16)))
    return static_cast<int>(hipErrorInvalidValue);
  const Riders rd{static_cast<const bf16_t*>(a_add), nullptr, nullptr};
  const RopeEpi rp{positions, seq_of_token, cos_t, sin_t, block_table,
                   static_cast<bf16_t*>(k_pages), static_cast<bf16_t*>(v_pages), H, KV, d, rot,
                   table_len, block_size, table_stride, num_blocks, write_kv, n_seqs};
  const int N = (H + 2 * KV) * d;
  const bf16_t* w = static_cast<const bf16_t*>(W);
  if (a_type == 0) return launch_rows<0, 4>(A, w, q_out, M, N, K, lda, ldq, eps, w_tiled, rd, rp, s);
  if (a_type == 1) return launch_rows<1, 4>(A, w, q_out, M, N, K, lda, ldq, eps, w_tiled, rd, rp, s);
  return static_cast<int>(hipErrorInvalidValue);
}


// How many workgroups the greedy pick of M rows over N columns launches: the caller sizes
// part_val / part_idx as 16 * that many.
KVF_EXPORT int kvf_gemm_bf16_pick_ticket_ints() { return PICK_TICKET_INTS; }
KVF_EXPORT int kvf_gemm_bf16_pick_groups(int M, int N) {
  const int tiles = (N + 15) / 16;
  const int nt = (M > 4 && tiles >= 512) ? 2 : 1;
  return (N + 16 * nt - 1) / (16 * nt);
}

// Output head of a decode step with the greedy pick and the step's tail folded in (EPI 5 at the
// head of the file).  A: the normalised rows [M <= 16, lda] bf16.  W: [N, K] bf16, row-major or
// tiled.  residual: [M, ld_res] fp32, receives the picked tokens' rows of `embed` [>= N, hidden].
// See PickEpi for the rest.
KVF_EXPORT int kvf_gemm_bf16_pick(const void* A, const void* W, int w_tiled, int M, int N, int K,
                                  int lda, float* part_val, int* part_idx, int* ticket, int* tokens,
                                  int* token_ids, int* positions, int* ctx_lens, int* ring,
                                  int* run_counter, int ring_stride, int ring_rows, const void* embed,
                                  float* residual, int hidden, int ld_res, hipStream_t s) {
  if (M <= 0) return 0;
  if (M > 16 || N <= 0 || K <= 0 || K % 8 != 0 || lda % 8 != 0 || hidden % 8 != 0 || ld_res % 4 != 0 ||
      ring_stride < M || ring_rows <= 0 || !part_val || !part_idx || !ticket)
    return static_cast<int>(hipErrorInvalidValue);
  const Riders rd{nullptr, nullptr, nullptr};
  const RopeEpi none{};
  const PickEpi pk{part_val, part_idx, ticket, tokens, token_ids, positions, ctx_lens, ring, run_counter,
                   static_cast<const bf16_t*>(embed), residual, ring_stride, ring_rows, hidden, ld_res};
  const bf16_t* w = static_cast<const bf16_t*>(W);
  if (M > 4 && (N + 15) / 16 >= 512)   // two groups of 16 columns per workgroup, as pick_groups counts
    return launch_one<1, 2, 0, 5>(A, w, nullptr, M, N, K, lda, 0, 0, 0.f, w_tiled, rd, none, s, pk);
  return launch_one<1, 1, 0, 5>(A, w, nullptr, M, N, K, lda, 0, 0, 0.f, w_tiled, rd, none, s, pk);
}
