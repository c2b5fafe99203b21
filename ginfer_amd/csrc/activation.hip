// SwiGLU on the fused gate-up product: out[t, i] = (g * (1 / (1 + exp(-g)))) * u with
// g = gu[t, i], u = gu[t, I + i].  32-bit arithmetic, one rounding.
// Formula: ginfer/core/op/kernels/cuda/swiglu_kernel.cu:24-27 (which skips a tail of numel % 8).
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

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

// The same on a product that lies transposed, gu_t [2 I, tokens] (a row holds one column of the product for all
// tokens): out [tokens, I].  The BLAS library's product with the weights as its first operand, which leaves this
// layout, is the faster one at some sizes.  A workgroup takes 64 columns x 64 tokens: 16-byte reads along the tokens,
// the activation in 32-bit, a turn through LDS, 16-byte writes along the columns.  bfloat16, tokens and I multiples of 8.
#define ST_TILE 64
__global__ __launch_bounds__(256) void silu_mul_transposed_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu_t,
                                                                  int tokens, int inter) {
  __shared__ bf16_t tile[ST_TILE][ST_TILE + 8];      // [token][column], rows 16-byte aligned
  const int i0 = blockIdx.x * ST_TILE, t0 = blockIdx.y * ST_TILE;
  {
    // a thread takes two neighbouring columns and 8 tokens: neighbouring lanes take neighbouring pairs of columns, so
    // their 32-bit writes into the tile fall into different banks
    const int il = (threadIdx.x % (ST_TILE / 2)) * 2, tl = (threadIdx.x / (ST_TILE / 2)) * 8;
    const int i = i0 + il, t = t0 + tl;
    if (i < inter && t < tokens) {                    // both are multiples of 8: a piece lies inside or outside
      union { uint4 v; bf16_t e[8]; } g[2], u[2];
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        g[c].v = *reinterpret_cast<const uint4*>(gu_t + (int64_t)(i + c) * tokens + t);
        u[c].v = *reinterpret_cast<const uint4*>(gu_t + (int64_t)(inter + i + c) * tokens + t);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        uint32_t pair = 0;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          const float gv = bf16_to_f32(g[c].e[j]), uv = bf16_to_f32(u[c].e[j]);
          pair |= (uint32_t)f32_to_bf16((gv * (1.0f / (1.0f + expf(-gv)))) * uv) << (16 * c);
        }
        *reinterpret_cast<uint32_t*>(&tile[tl + j][il]) = pair;
      }
    }
  }
  __syncthreads();
  for (int item = threadIdx.x; item < ST_TILE * (ST_TILE / 8); item += 256) {
    const int tl = item / (ST_TILE / 8), il = (item % (ST_TILE / 8)) * 8;
    const int t = t0 + tl, i = i0 + il;
    if (t >= tokens || i >= inter) continue;
    *reinterpret_cast<uint4*>(out + (int64_t)t * inter + i) = *reinterpret_cast<const uint4*>(&tile[tl][il]);
  }
}

// out [tokens, inter] bfloat16; gu_t [2 * inter, tokens] bfloat16 contiguous; tokens and inter multiples of 8.
extern "C" int ga_silu_mul_transposed(void* out, const void* gu_t, int tokens, int inter, hipStream_t stream) {
  if (tokens <= 0 || inter <= 0) return 0;
  if (tokens % 8 || inter % 8) return -1;
  dim3 grid((inter + ST_TILE - 1) / ST_TILE, (tokens + ST_TILE - 1) / ST_TILE), block(256);
  if (grid.y > 65535) return -2;
  hipLaunchKernelGGL(silu_mul_transposed_kernel, grid, block, 0, stream, (bf16_t*)out, (const bf16_t*)gu_t, tokens, inter);
  return GA_CHECK_LAUNCH();
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
