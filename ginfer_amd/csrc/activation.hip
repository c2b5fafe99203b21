// SwiGLU on the fused gate-up product: out[t, i] = (g * (1 / (1 + exp(-g)))) * u with
// g = gu[t, i], u = gu[t, I + i].  32-bit arithmetic, one rounding.
// Formula: ginfer/core/op/kernels/cuda/swiglu_kernel.cu:24-27 (which skips a tail of numel % 8).
#include "common.cuh"

template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t tokens,
                                int inter) {
  const int64_t total = tokens * inter;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / inter;
    const int i = (int)(idx - t * inter);
    const float g = Num<T>::ld(gu + t * 2 * inter + i);
    const float u = Num<T>::ld(gu + t * 2 * inter + inter + i);
    const float sig = 1.0f / (1.0f + expf(-g));
    Num<T>::st(out + idx, (g * sig) * u);
  }
}

// eight elements to a thread in 16-byte accesses, for I a multiple of 8
template <typename T>
__global__ void silu_mul_vec_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t tokens, int inter) {
  constexpr int V = 16 / sizeof(T);
  const int chunks = inter / V;
  const int64_t total = tokens * chunks;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / chunks;
    const int i = (int)(idx - t * chunks) * V;
    union { uint4 u; T e[V]; } g, u, o;
    g.u = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + i);
    u.u = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + inter + i);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float gv = Num<T>::ld(&g.e[j]), uv = Num<T>::ld(&u.e[j]);
      const float sig = 1.0f / (1.0f + expf(-gv));
      Num<T>::st(&o.e[j], (gv * sig) * uv);
    }
    *reinterpret_cast<uint4*>(out + t * inter + i) = o.u;
  }
}

extern "C" int ga_silu_mul(void* out, const void* gu, int tokens, int inter, int is_bf16,
                           hipStream_t stream) {
  if (tokens <= 0) return 0;
  int64_t total = (int64_t)tokens * inter;
  if (inter % 8 == 0) {
    const int v = is_bf16 ? 8 : 4;
    int64_t nb = (total / v + 255) / 256;
    dim3 vgrid((unsigned)(nb > 16384 ? 16384 : nb)), vblock(256);
    if (is_bf16)
      hipLaunchKernelGGL(silu_mul_vec_kernel<bf16_t>, vgrid, vblock, 0, stream, (bf16_t*)out, (const bf16_t*)gu,
                         (int64_t)tokens, inter);
    else
      hipLaunchKernelGGL(silu_mul_vec_kernel<float>, vgrid, vblock, 0, stream, (float*)out, (const float*)gu,
                         (int64_t)tokens, inter);
    return GA_CHECK_LAUNCH();
  }
  int blocks = (int)((total + 255) / 256);
  if (blocks > 65536) blocks = 65536;
  dim3 grid(blocks), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out,
                       (const bf16_t*)gu, (int64_t)tokens, inter);
  else
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (float*)out,
                       (const float*)gu, (int64_t)tokens, inter);
  return GA_CHECK_LAUNCH();
}
