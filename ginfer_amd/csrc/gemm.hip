// Matrix products C[M, N] = A[M, K] . W[N, K]^T (+ bias[N]) with W stored [out, in] row-major, the
// layout of the checkpoint (ginfer/core/layer/linear.cc:9-20); 32-bit accumulation and the bias
// added in 32-bit before the one rounding (ginfer/core/op/kernels/cuda/gemm_kernel/
// gemm_kernel.cu:100-121, ginfer/core/op/kernels/cuda/gemv_kernel.cu:52-55).
//
// gemm_nt_kernel is the true 32-bit product (plain FMA, no matrix unit, no reduced-precision
// mode): a tile of C per workgroup, staged through LDS in steps of K.  Every element of C is ONE accumulator
// summed over k in ascending order, so its bits do not depend on M, on the tile it falls in, on the tile's
// shape or on the rest of the batch: the two shapes below (64 x 64 for many rows, 16 x 32 for the few rows
// of a decode step, where only the columns can be shared out) give the same bits for the same row.  It is
// templated on storage so that it also serves bfloat16 operands (the kernel tests' oracle and the fallback
// for shapes the matrix-core kernels refuse).
//
// A step of K is asked for (in 16-byte loads where rows allow it, consecutive lanes on consecutive elements)
// while the step before is being multiplied: the loads' way from memory, which a workgroup of a decode step
// would otherwise wait out some hundred times in a row, runs beside the arithmetic.
#include "common.cuh"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

#define GEMM_THREADS 256

// four consecutive elements as floats; `wide`: one load (the address is a multiple of four elements)
template <typename T>
__device__ __forceinline__ void load4(float (&v)[4], const T* p, int valid, bool wide);
template <>
__device__ __forceinline__ void load4<float>(float (&v)[4], const float* p, int valid, bool wide) {
  if (wide && valid == 4) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = i < valid ? p[i] : 0.f;
  }
}
template <>
__device__ __forceinline__ void load4<bf16_t>(float (&v)[4], const bf16_t* p, int valid, bool wide) {
  if (wide && valid == 4) {
    const uint2 x = *reinterpret_cast<const uint2*>(p);
    v[0] = bf16_to_f32((bf16_t)(x.x & 0xffffu)); v[1] = bf16_to_f32((bf16_t)(x.x >> 16));
    v[2] = bf16_to_f32((bf16_t)(x.y & 0xffffu)); v[3] = bf16_to_f32((bf16_t)(x.y >> 16));
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = i < valid ? bf16_to_f32(p[i]) : 0.f;
  }
}

// TM x TN: the workgroup's tile of C; TK: elements of K per step; a thread owns RM x RN elements, the threads
// lie 16 x 16 over the tile (TM = 16 RM, TN = 16 RN).
template <typename TA, typename TW, typename TC, int TM, int TN, int TK>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_nt_kernel(TC* __restrict__ C, int64_t ldc,
                                                               const TA* __restrict__ A, int64_t lda,
                                                               const TW* __restrict__ W,
                                                               const TW* __restrict__ bias, int M, int N,
                                                               int K, int wide_a, int wide_w) {
  constexpr int RM = TM / 16, RN = TN / 16;
  constexpr int GA = TM * TK / 4 / GEMM_THREADS, GW = TN * TK / 4 / GEMM_THREADS;     // groups of four per thread
  static_assert(GA >= 1 && GW >= 1 && TM % 16 == 0 && TN % 16 == 0, "tile sizes");
  __shared__ float a_s[TK][TM + 4];
  __shared__ float w_s[TK][TN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int tx = tid % 16, ty = tid / 16;  // the thread's block: rows ty*RM.., columns tx*RN..
  float acc[RM][RN];
#pragma unroll
  for (int i = 0; i < RM; ++i)
#pragma unroll
    for (int j = 0; j < RN; ++j) acc[i][j] = 0.f;

  float ra[GA][4], rw[GW][4];
  // group number gi of a step: row gi / (TK / 4) of the tile, elements 4 (gi % (TK / 4)) .. + 3 of the step
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < GA; ++i) {
      const int gi = tid + i * GEMM_THREADS, row = gi / (TK / 4), k = k0 + (gi % (TK / 4)) * 4;
      const int m = m0 + row;
      const int valid = (m < M && k < K) ? (K - k < 4 ? K - k : 4) : 0;
      if (valid) load4<TA>(ra[i], A + (int64_t)m * lda + k, valid, wide_a != 0);
      else ra[i][0] = ra[i][1] = ra[i][2] = ra[i][3] = 0.f;
    }
#pragma unroll
    for (int i = 0; i < GW; ++i) {
      const int gi = tid + i * GEMM_THREADS, row = gi / (TK / 4), k = k0 + (gi % (TK / 4)) * 4;
      const int n = n0 + row;
      const int valid = (n < N && k < K) ? (K - k < 4 ? K - k : 4) : 0;
      if (valid) load4<TW>(rw[i], W + (int64_t)n * K + k, valid, wide_w != 0);
      else rw[i][0] = rw[i][1] = rw[i][2] = rw[i][3] = 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < GA; ++i) {
      const int gi = tid + i * GEMM_THREADS, row = gi / (TK / 4), kk = (gi % (TK / 4)) * 4;
#pragma unroll
      for (int j = 0; j < 4; ++j) a_s[kk + j][row] = ra[i][j];
    }
#pragma unroll
    for (int i = 0; i < GW; ++i) {
      const int gi = tid + i * GEMM_THREADS, row = gi / (TK / 4), kk = (gi % (TK / 4)) * 4;
#pragma unroll
      for (int j = 0; j < 4; ++j) w_s[kk + j][row] = rw[i][j];
    }
    __syncthreads();
    if (k0 + TK < K) fetch(k0 + TK);        // on its way while this step is multiplied
#pragma unroll 8
    for (int k = 0; k < TK; ++k) {
      float a[RM], w[RN];
#pragma unroll
      for (int i = 0; i < RM; ++i) a[i] = a_s[k][ty * RM + i];
#pragma unroll
      for (int j = 0; j < RN; ++j) w[j] = w_s[k][tx * RN + j];
#pragma unroll
      for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int j = 0; j < RN; ++j) acc[i][j] = __builtin_fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < RM; ++i) {
    const int m = m0 + ty * RM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < RN; ++j) {
      const int n = n0 + tx * RN + j;
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
  const bool few = M <= 16;                 // a decode step's rows: 16 x 32 tiles, long steps of K
  const int tm = few ? 16 : 64, tn = few ? 32 : 64;
  dim3 grid((N + tn - 1) / tn, (M + tm - 1) / tm), block(GEMM_THREADS);
  if (grid.y > 65535) return -2;
  // 16-byte loads (8 bytes for bfloat16) need rows that start at multiples of four elements
  const size_t unit = in_bf16 ? 8 : 16;
  const int wide_a = (K % 4 == 0 && lda % 4 == 0 && (uintptr_t)A % unit == 0) ? 1 : 0;
  const int wide_w = (K % 4 == 0 && (uintptr_t)W % unit == 0) ? 1 : 0;
#define LAUNCH(TA, TW, TC)                                                                                   \
  do {                                                                                                       \
    if (few)                                                                                                 \
      hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, TC, 16, 32, 128>), grid, block, 0, stream, (TC*)C, ldc,     \
                         (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a, wide_w);         \
    else                                                                                                     \
      hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, TC, 64, 64, 32>), grid, block, 0, stream, (TC*)C, ldc,      \
                         (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a, wide_w);         \
  } while (0)
  if (in_bf16) {
    if (out_bf16) LAUNCH(bf16_t, bf16_t, bf16_t); else LAUNCH(bf16_t, bf16_t, float);
  } else {
    if (out_bf16) return -3;
    LAUNCH(float, float, float);
  }
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
