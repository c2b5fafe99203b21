// Filling a tensor with normal numbers on the device: element i = mean + std * normal(key, i), the generator of
// random_normal.h, which the host library random_fill_host.cpp shares: the same seed gives the same bits on both.
// For models too large to pass through a file (a 72B shape is 145 GB of weights).
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations
#include "random_normal.h"

#define FILL_THREADS 256

template <typename T>
__global__ __launch_bounds__(FILL_THREADS) void random_normal_fill_kernel(T* __restrict__ out, int64_t n, uint64_t key,
                                                                           float mean, float std) {
  const int64_t stride = (int64_t)gridDim.x * FILL_THREADS;
  for (int64_t i = (int64_t)blockIdx.x * FILL_THREADS + threadIdx.x; i < n; i += stride)
    Num<T>::st(out + i, ga_weight_from_counter(key, (uint64_t)i, mean, std));
}

// out: n elements, float or bfloat16 (rounded to nearest even from the 32-bit number)
extern "C" int ga_random_normal_fill(void* out, int64_t n, uint64_t key, float mean, float std, int is_bf16,
                                     hipStream_t stream) {
  if (n <= 0) return 0;
  if (!out) return -1;
  int64_t blocks = (n + FILL_THREADS - 1) / FILL_THREADS;
  if (blocks > 256 * 32) blocks = 256 * 32;
  if (is_bf16)
    hipLaunchKernelGGL(random_normal_fill_kernel<bf16_t>, dim3((unsigned)blocks), dim3(FILL_THREADS), 0, stream,
                       (bf16_t*)out, n, key, mean, std);
  else
    hipLaunchKernelGGL(random_normal_fill_kernel<float>, dim3((unsigned)blocks), dim3(FILL_THREADS), 0, stream,
                       (float*)out, n, key, mean, std);
  return GA_CHECK_LAUNCH();
}
