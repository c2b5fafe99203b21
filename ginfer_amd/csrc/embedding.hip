// Token embedding gather: residual[t, :] = (float) table[ids[t], :].
// The residual stream is kept in 32-bit in both dtypes, so the gather widens as it copies.
// Formula: ginfer/core/op/kernels/cuda/embedding_kernel.cu:16-24 (which copies in the table's
// dtype and drops a tail of H % 8 elements; here every element is copied).
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

template <typename T>
__global__ void embedding_gather_kernel(float* __restrict__ out, const T* __restrict__ table,
                                        const int32_t* __restrict__ ids, int hidden) {
  const int64_t t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * hidden;
  float* o = out + t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = Num<T>::ld(row + i);
}

extern "C" int ga_embedding_gather(void* out, const void* table, const void* ids, int tokens,
                                   int hidden, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  dim3 grid(tokens), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(embedding_gather_kernel<bf16_t>, grid, block, 0, stream, (float*)out,
                       (const bf16_t*)table, (const int32_t*)ids, hidden);
  else
    hipLaunchKernelGGL(embedding_gather_kernel<float>, grid, block, 0, stream, (float*)out,
                       (const float*)table, (const int32_t*)ids, hidden);
  return GA_CHECK_LAUNCH();
}
