// Fused residual add + RMSNorm.
//   h = residual[t] + delta[t]        (32-bit add; written back to the 32-bit residual stream)
//   y = (h * g) / sqrt(sum(h^2)/H + eps)
// Formula and order of operations: ginfer/core/op/kernels/cuda/rmsnorm_kernel.cu:27-66 (sum :31-44,
// rms :54, (x*g)/rms :63); the add replaces ginfer/core/op/kernels/cuda/add_kernel.cu:10-35, which
// adds in 16-bit.  With `rows` the kernel normalises only the listed rows (the gather before the
// output head, ginfer/core/op/kernels/cuda/select_last_token_kernel.cu:8-27) and leaves the
// residual stream untouched, so a row may be listed twice.
// The sum over a row is taken in a fixed order that depends on H alone, so a row's result does not
// depend on which other rows are in the batch.
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

#define NORM_THREADS 256

// D is the type of delta: the compute dtype, or float when delta holds `parts` partial sums of a
// K-split matrix product ([parts][T][H]); the parts are added in order, after one another.
template <typename T, typename G, typename D>
__global__ void add_rmsnorm_kernel(T* __restrict__ out, float* __restrict__ residual,
                                   const D* __restrict__ delta, int parts, int64_t part_stride,
                                   const G* __restrict__ gain, const int32_t* __restrict__ rows, int hidden,
                                   float eps) {
  __shared__ float scratch[NORM_THREADS / WAVE];
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? (int64_t)rows[r] : r;
  float* res = residual + t * hidden;
  const D* d = delta ? delta + t * hidden : nullptr;
  const bool write_back = (rows == nullptr) && (d != nullptr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += NORM_THREADS) {
    float h = res[i];
    if (d) {
      float add = Num<D>::ld(d + i);
      for (int p = 1; p < parts; ++p) add += Num<D>::ld(d + p * part_stride + i);
      h += add;
    }
    if (write_back) res[i] = h;
    ss += h * h;
  }
  ss = block_sum<NORM_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps);
  T* o = out + r * hidden;
  for (int i = threadIdx.x; i < hidden; i += NORM_THREADS) {
    float h = res[i];                       // own write of the first pass when write_back
    if (d && !write_back) {
      float add = Num<D>::ld(d + i);
      for (int p = 1; p < parts; ++p) add += Num<D>::ld(d + p * part_stride + i);
      h += add;
    }
    Num<T>::st(o + i, (h * Num<G>::ld(gain + i)) / rms);
  }
}

// The same, eight elements to a thread in 16-byte accesses, the row kept in registers between the sum
// and the scaling; for H a multiple of 8 up to 8 * NORM_THREADS * VEC_CHUNKS.  The sum over the row adds
// each thread's elements in ascending order and then the threads in the fixed order of block_sum, so it
// too depends on H alone.
#define VEC_CHUNKS 4

template <typename D>
__device__ __forceinline__ void load8f(float (&v)[8], const D* p);
template <>
__device__ __forceinline__ void load8f<float>(float (&v)[8], const float* p) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <>
__device__ __forceinline__ void load8f<bf16_t>(float (&v)[8], const bf16_t* p) {
  const uint4 u = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
template <typename T>
__device__ __forceinline__ void store8f(T* p, const float (&v)[8]);
template <>
__device__ __forceinline__ void store8f<float>(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <>
__device__ __forceinline__ void store8f<bf16_t>(bf16_t* p, const float (&v)[8]) {
  uint4 u;
  u.x = f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
  u.y = f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
  u.z = f32_to_bf16(v[4]) | ((uint32_t)f32_to_bf16(v[5]) << 16);
  u.w = f32_to_bf16(v[6]) | ((uint32_t)f32_to_bf16(v[7]) << 16);
  *reinterpret_cast<uint4*>(p) = u;
}

template <typename T, typename G, typename D, int PARTS /* 0: runtime */>
__global__ __launch_bounds__(NORM_THREADS) void add_rmsnorm_vec_kernel(
    T* __restrict__ out, float* __restrict__ residual, const D* __restrict__ delta, int parts_rt,
    int64_t part_stride, const G* __restrict__ gain, const int32_t* __restrict__ rows, int hidden, float eps) {
  __shared__ float scratch[NORM_THREADS / WAVE];
  const int parts = PARTS ? PARTS : parts_rt;
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? (int64_t)rows[r] : r;
  float* res = residual + t * hidden;
  const D* d = delta ? delta + t * hidden : nullptr;
  const bool write_back = (rows == nullptr) && (d != nullptr);
  float h[VEC_CHUNKS][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < VEC_CHUNKS; ++c) {
    const int i = (c * NORM_THREADS + threadIdx.x) * 8;
    if (i < hidden) {
      load8f<float>(h[c], res + i);
      if (d) {
        float add[8];
        load8f<D>(add, d + i);
        for (int p = 1; p < parts; ++p) {
          float more[8];
          load8f<D>(more, d + p * part_stride + i);
#pragma unroll
          for (int j = 0; j < 8; ++j) add[j] += more[j];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) h[c][j] += add[j];
        if (write_back) store8f<float>(res + i, h[c]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += h[c][j] * h[c][j];
    }
  }
  ss = block_sum<NORM_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps);
  T* o = out + r * hidden;
#pragma unroll
  for (int c = 0; c < VEC_CHUNKS; ++c) {
    const int i = (c * NORM_THREADS + threadIdx.x) * 8;
    if (i < hidden) {
      float g[8], y[8];
      load8f<G>(g, gain + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = (h[c][j] * g[j]) / rms;
      store8f<T>(o + i, y);
    }
  }
}

// out: [R, H] in the compute dtype; residual: [T, H] float; delta: [T, H] compute dtype or null, or, with
// delta_parts > 0, float [delta_parts][T][H] partial sums; gain: [H] compute dtype, or float when
// gain_is_f32; rows: [R] int32 or null (then R == T); num_tokens = T.
extern "C" int ga_add_rmsnorm(void* out, void* residual, const void* delta, int delta_parts, int num_tokens,
                              const void* gain, const void* rows, int num_rows, int hidden, float eps,
                              int is_bf16, int gain_is_f32, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  dim3 grid(num_rows), block(NORM_THREADS);
  const int64_t stride = (int64_t)num_tokens * hidden;
  if (hidden % 8 == 0 && hidden <= 8 * NORM_THREADS * VEC_CHUNKS) {
#define VLAUNCH(T, G, D, P)                                                                          \
  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, G, D, P>), grid, block, 0, stream, (T*)out,         \
                     (float*)residual, (const D*)delta, delta_parts, stride, (const G*)gain,         \
                     (const int32_t*)rows, hidden, eps)
#define VPARTS(T, G)                                                                                 \
  if (delta_parts == 4) VLAUNCH(T, G, float, 4); else if (delta_parts == 2) VLAUNCH(T, G, float, 2); \
  else if (delta_parts == 8) VLAUNCH(T, G, float, 8); else VLAUNCH(T, G, float, 0)
    if (delta_parts > 0) {
      if (is_bf16) {
        if (gain_is_f32) { VPARTS(bf16_t, float); } else { VPARTS(bf16_t, bf16_t); }
      } else {
        VPARTS(float, float);
      }
    } else if (is_bf16) {
      if (gain_is_f32) VLAUNCH(bf16_t, float, bf16_t, 1); else VLAUNCH(bf16_t, bf16_t, bf16_t, 1);
    } else {
      VLAUNCH(float, float, float, 1);
    }
#undef VPARTS
#undef VLAUNCH
    return GA_CHECK_LAUNCH();
  }
#define LAUNCH(T, G, D, PARTS)                                                                    \
  hipLaunchKernelGGL((add_rmsnorm_kernel<T, G, D>), grid, block, 0, stream, (T*)out,             \
                     (float*)residual, (const D*)delta, PARTS, stride, (const G*)gain,            \
                     (const int32_t*)rows, hidden, eps)
  if (delta_parts > 0) {
    if (is_bf16) {
      if (gain_is_f32) LAUNCH(bf16_t, float, float, delta_parts); else LAUNCH(bf16_t, bf16_t, float, delta_parts);
    } else {
      LAUNCH(float, float, float, delta_parts);
    }
  } else if (is_bf16) {
    if (gain_is_f32) LAUNCH(bf16_t, float, bf16_t, 1); else LAUNCH(bf16_t, bf16_t, bf16_t, 1);
  } else {
    LAUNCH(float, float, float, 1);
  }
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
