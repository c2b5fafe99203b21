// Shared device helpers for the gfx950 kernels: 64-wide wavefront reductions, bf16 <-> fp32, and
// typed loads that always hand the arithmetic a float.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;  // raw bfloat16 bits

#define WAVE 64

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

template <typename T> struct Num;
template <> struct Num<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Num<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};

// butterfly reductions over the 64 lanes of a wavefront: every lane ends with the same value, and
// the order of the additions is the same whatever the data
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// sum over a workgroup of NWAVES wavefronts; `scratch` holds NWAVES floats of LDS
template <int NWAVES>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NWAVES; ++i) t += scratch[i];
  return t;
}

#define GA_CHECK_LAUNCH() ((int)hipGetLastError())

// Page and place in the page of a cache slot (slot >= 0).  Page sizes are powers of two nearly always: then a shift,
// for a 64-bit division is some hundred instructions, in every thread, before the first store can go out.
__device__ __forceinline__ void slot_page(int64_t slot, int page_size, int64_t& page, int64_t& off) {
  if ((page_size & (page_size - 1)) == 0) page = slot >> (__ffs(page_size) - 1);
  else page = slot / page_size;
  off = slot - page * page_size;
}
