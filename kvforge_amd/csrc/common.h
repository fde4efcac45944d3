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

// round to nearest even, NaN kept quiet
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
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
