// Shared helpers for the gfx950 kernels: element types, conversions, wave reductions.
// Every exported function has C linkage, takes raw device pointers plus a hipStream_t and
// returns a hipError_t code as int (0 = success).  Shapes are validated by the Python caller
// before launch; kernels additionally guard every index that comes from device data
// (token ids, page numbers) so that bad data yields skipped work, never a stray access.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define KVF_EXPORT extern "C" __attribute__((visibility("default")))
#define KVF_WAVE 64

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// round to nearest even (the hardware conversion of gfx950)
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(p->bits); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { p->bits = f32_to_bf16(v); }
};

// load 8 consecutive elements as floats; p must be 16-byte (bf16) / 32-byte (float) aligned
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
  const uint4 r = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// Sum over aligned groups of G neighbouring lanes (G = 2..32), left in every lane of the group.
// Data-parallel-primitive moves ride in the add itself; only the 32-lane step crosses a row
// of 16 and needs the LDS crossbar.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int G> __device__ __forceinline__ float group_sum(float v) {
  static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16 || G == 32, "group size");
  if (G >= 2) v += dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]: lane ^ 1
  if (G >= 4) v += dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]: lane ^ 2
  if (G >= 8) v += dpp_move<0x141>(v);   // row_half_mirror: the other quad of 8 lanes
  if (G >= 16) v += dpp_move<0x140>(v);  // row_mirror: the other half of 16 lanes
  if (G >= 32) v += __shfl_xor(v, 16, KVF_WAVE);
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = KVF_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, KVF_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = KVF_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, KVF_WAVE));
  return v;
}

// block-wide sum for blocks of up to 1024 threads; `scratch` holds >= 16 floats of LDS
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int nwaves = (blockDim.x + KVF_WAVE - 1) / KVF_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

static inline int kvf_last_error() { return static_cast<int>(hipGetLastError()); }
