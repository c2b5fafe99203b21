// C[M, N] = A[M, K] . W[N, K]^T (+ bias) for FEW rows (M <= 64): the decode step's products, where
// every weight is read once and the time is the weight's way from HBM.  bfloat16 operands, 32-bit
// accumulation on the matrix cores, bias added in 32-bit before the one rounding (the reference's
// small-batch kernel is ginfer/core/op/kernels/cuda/gemv_kernel.cu:13-58: one block per output column,
// scalar FMAs; its engine never reaches it, ginfer/core/op/matmul_op.cc:47-50).
//
// A workgroup of 8 wavefronts owns NT*16 rows of W (output columns) and all M rows of A; the wavefronts
// split K and add their parts up through LDS in a fixed order.  v_mfma_f32_16x16x32_bf16 with W as the
// first operand: lane l supplies W[n0 + l%16][k-slots] and A[l%16][k-slots] and receives
// D[n = (l/16)*4+i][m = l%16].  Both operands come straight from global memory in 16-byte loads, no LDS
// staging: the k-slots of a lane are 8 consecutive elements, and since a sum over k may take its terms
// in any order as long as both operands agree, lane group g = l/16 takes the 16 elements
// [k + 16g, k + 16g + 16) of every 64-element step as two products, so that the four lanes of a row read
// 128 consecutive bytes.
#include "common.cuh"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define SK_WAVES 8
#define SK_THREADS (SK_WAVES * 64)

__device__ __forceinline__ bf16x8 zero8() {
  uint4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}
__device__ __forceinline__ bf16x8 load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

template <int NT, int MB, typename TC>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(TC* __restrict__ C, int64_t ldc,
                                                                 const bf16_t* __restrict__ A, int64_t lda,
                                                                 const bf16_t* __restrict__ W,
                                                                 const bf16_t* __restrict__ bias, int M, int N,
                                                                 int K, int kchunk) {
  __shared__ float red[SK_WAVES][NT * 16][MB * 16 + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * NT * 16;
  const int kb = wave * kchunk;
  const int ke = kb + kchunk < K ? kb + kchunk : K;

  const bf16_t* wp[NT];
  bool wok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = n0 + nt * 16 + r;
    wok[nt] = n < N;
    wp[nt] = W + (int64_t)(wok[nt] ? n : 0) * K;
  }
  const bf16_t* ap[MB];
  bool aok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + r;
    aok[mb] = m < M;
    ap[mb] = A + (int64_t)(aok[mb] ? m : 0) * lda;
  }
  f32x4 acc[NT][MB];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll 2
  for (int k = kb; k < ke; k += 64) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int kk = k + g * 16 + j * 8;
      const bool ok = kk < ke;
      bf16x8 a[NT], b[MB];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) a[nt] = (ok && wok[nt]) ? load8(wp[nt] + kk) : zero8();
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) b[mb] = (ok && aok[mb]) ? load8(ap[mb] + kk) : zero8();
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[nt][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt], b[mb], acc[nt][mb], 0, 0, 0);
    }
  }
  // parts of the K-split meet in LDS and are added in wavefront order
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][nt * 16 + g * 4 + i][mb * 16 + r] = acc[nt][mb][i];
  __syncthreads();
  for (int idx = threadIdx.x; idx < NT * 16 * MB * 16; idx += SK_THREADS) {
    const int nl = idx % (NT * 16), m = idx / (NT * 16);
    const int n = n0 + nl;
    if (m >= M || n >= N) continue;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < SK_WAVES; ++w) v += red[w][nl][m];
    if (bias) v += bf16_to_f32(bias[n]);
    Num<TC>::st(C + (int64_t)m * ldc + n, v);
  }
}

// A [M, K] (row stride lda), W [N, K] contiguous, bias [N] or null, C [M, N] (row stride ldc) in
// bfloat16 or float.  M <= 64, K a multiple of 8, rows 16-byte aligned.
extern "C" int ga_gemm_skinny(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias,
                              int M, int N, int K, int out_f32, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 || lda % 8) return -1;
  const int mb = (M + 15) / 16;
  const int nt = N >= 4096 ? 2 : 1;
  int kchunk = ((K + SK_WAVES - 1) / SK_WAVES + 63) / 64 * 64;
  dim3 grid((N + nt * 16 - 1) / (nt * 16)), block(SK_THREADS);
#define LAUNCH(NT, MB, TC)                                                                              \
  hipLaunchKernelGGL((gemm_skinny_kernel<NT, MB, TC>), grid, block, 0, stream, (TC*)C, ldc,            \
                     (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, M, N, K, kchunk)
#define PICK_MB(NT, TC)                                                                                 \
  switch (mb) {                                                                                         \
    case 1: LAUNCH(NT, 1, TC); break;                                                                   \
    case 2: LAUNCH(NT, 2, TC); break;                                                                   \
    case 3: LAUNCH(NT, 3, TC); break;                                                                   \
    default: LAUNCH(NT, 4, TC); break;                                                                  \
  }
  if (out_f32) {
    if (nt == 2) { PICK_MB(2, float) } else { PICK_MB(1, float) }
  } else {
    if (nt == 2) { PICK_MB(2, bf16_t) } else { PICK_MB(1, bf16_t) }
  }
#undef PICK_MB
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
