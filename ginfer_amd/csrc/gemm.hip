// Matrix products C[M, N] = A[M, K] . W[N, K]^T (+ bias[N]) with W stored [out, in] row-major, the
// layout of the checkpoint (ginfer/core/layer/linear.cc:9-20); 32-bit accumulation and the bias
// added in 32-bit before the one rounding (ginfer/core/op/kernels/cuda/gemm_kernel/
// gemm_kernel.cu:100-121, ginfer/core/op/kernels/cuda/gemv_kernel.cu:52-55).
//
// gemm_nt_kernel is the true 32-bit product (plain FMA, no matrix unit, no reduced-precision
// mode): a 64x64 tile per workgroup staged through LDS in K-steps of 16, a 4x4 block per thread.
// Every element of C is one accumulator summed over k in ascending order, so its bits do not
// depend on M, on the tile it falls in or on the rest of the batch.  It is templated on storage so
// that it also serves bfloat16 operands (the kernel tests' oracle and the fallback for shapes the
// matrix-core kernels refuse).
#include "common.cuh"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

#define TM 64
#define TN 64
#define TK 16

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_kernel(TC* __restrict__ C, int64_t ldc,
                                                      const TA* __restrict__ A, int64_t lda,
                                                      const TW* __restrict__ W,
                                                      const TW* __restrict__ bias, int M, int N,
                                                      int K) {
  __shared__ float a_s[TK][TM + 4];
  __shared__ float w_s[TK][TN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int tx = tid % 16, ty = tid / 16;  // thread's 4x4 block: rows ty*4.., cols tx*4..
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // each thread stages 4 elements of A and 4 of W per K-step: row = tid / 4, k = (tid % 4) * 4 ..
  const int lr = tid / 4, lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      const int m = m0 + lr, n = n0 + lr;
      a_s[lk + i][lr] = (m < M && k < K) ? Num<TA>::ld(A + (int64_t)m * lda + k) : 0.f;
      w_s[lk + i][lr] = (n < N && k < K) ? Num<TW>::ld(W + (int64_t)n * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = a_s[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = w_s[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * w[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += Num<TW>::ld(bias + n);
      Num<TC>::st(C + (int64_t)m * ldc + n, v);
    }
  }
}

// in_bf16: A, W and bias are bfloat16 (else float); out_bf16: C is bfloat16 (else float).
extern "C" int ga_gemm_nt(void* C, int64_t ldc, const void* A, int64_t lda, const void* W,
                          const void* bias, int M, int N, int K, int in_bf16, int out_bf16,
                          hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return -1;
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM), block(256);
  if (grid.y > 65535) return -2;
#define LAUNCH(TA, TW, TC)                                                                        \
  hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, TC>), grid, block, 0, stream, (TC*)C, ldc,          \
                     (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K)
  if (in_bf16) {
    if (out_bf16) LAUNCH(bf16_t, bf16_t, bf16_t); else LAUNCH(bf16_t, bf16_t, float);
  } else {
    if (out_bf16) return -3;
    LAUNCH(float, float, float);
  }
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
