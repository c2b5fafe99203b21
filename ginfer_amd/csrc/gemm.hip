// Matrix products C[M, N] = A[M, K] . W[N, K]^T (+ bias[N]) with W stored [out, in] row-major, the
// layout of the checkpoint (ginfer/core/layer/linear.cc:9-20); 32-bit accumulation and the bias
// added in 32-bit before the one rounding (ginfer/core/op/kernels/cuda/gemm_kernel/
// gemm_kernel.cu:100-121, ginfer/core/op/kernels/cuda/gemv_kernel.cu:52-55).
//
// Three kernels make the true 32-bit product (no reduced-precision mode anywhere).  In all of them every element of
// C is ONE accumulator that takes its terms over ascending k as fused multiply-adds, so its bits do not depend on M,
// on the tile it falls in, on the rest of the batch, or on which of the three ran:
//   gemm_nt_few_rows_kernel  up to 64 rows (a decode step, a small portion): the matrix cores' 32-bit instruction, a
//                            wavefront per 16 columns and up to four blocks of 16 rows, operands straight from memory;
//   gemm_nt_matrix_kernel    more rows: the matrix cores again, over tiles of up to 128 x 128 through LDS;
//   gemm_nt_kernel           plain FMA, a tile of 64 x 64 per workgroup staged through LDS in steps of K: 33 to 64 rows
//                            times 65,536 columns and more (a head), where it is the fastest of the three.
// They are templated on storage, so that they also serve bfloat16 operands (the kernel tests' oracle and the
// fallback for shapes the bfloat16 kernels refuse).
//
// A step of K is asked for (in 16-byte loads where rows allow it, consecutive lanes on consecutive elements)
// while the step before is being multiplied.
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

#define GEMM_THREADS 256
#ifndef GEMM_MATRIX_FROM_ROWS
#define GEMM_MATRIX_FROM_ROWS 64    // more rows than this: the kernel on the matrix cores (the same bits)
#endif

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

// The same product on the matrix cores, for many rows.  v_mfma_f32_32x32x2_f32 takes 32-bit operands and adds the two
// products of its step of K into the accumulator one after the other, each as a fused multiply-add: measured on the
// device, its results over a K of 512 equal the chain of fmaf over ascending k bit for bit, for every element of the
// tile.  So this kernel gives the bits of the kernel above at some three times its rate.  A workgroup of four
// wavefronts, 2 x 2 over a tile of TM x TN; a wavefront owns (TM / 2) x (TN / 2) as blocks of 32 x 32.  Lane l supplies
// row l % 32 of a block's A and W for k = step + l / 32 and receives, in register r, row 4 (l / 32) + 8 (r / 4) + r % 4
// and column l % 32 of the block.  Staging as above (k-major in LDS, the next step of K on its way meanwhile); rows
// are padded by two words so that the transposing stores of a wavefront fall into different banks.
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <typename TA, typename TW, typename TC, int TM, int TN, int TK>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_nt_matrix_kernel(TC* __restrict__ C, int64_t ldc,
                                                                      const TA* __restrict__ A, int64_t lda,
                                                                      const TW* __restrict__ W,
                                                                      const TW* __restrict__ bias, int M, int N,
                                                                      int K, int wide_a, int wide_w) {
  constexpr int BM = TM / 64, BN = TN / 64;         // blocks of 32 x 32 per wavefront, down and across
  constexpr int GA = TM * TK / 4 / GEMM_THREADS, GW = TN * TK / 4 / GEMM_THREADS;
  static_assert(GA >= 1 && GW >= 1 && TM % 64 == 0 && TN % 64 == 0 && TK % 2 == 0, "tile sizes");
  __shared__ float a_s[TK][TM + 2];
  __shared__ float w_s[TK][TN + 2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int wm = (wave >> 1) * (TM / 2), wn = (wave & 1) * (TN / 2);     // the wavefront's corner in the tile
  const int l32 = lane & 31, half = lane >> 5;
  f32x16 acc[BM][BN];
#pragma unroll
  for (int i = 0; i < BM; ++i)
#pragma unroll
    for (int j = 0; j < BN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  float ra[GA][4], rw[GW][4];
  // a tile that lies inside C, with rows that allow 16-byte loads, asks nothing per load while its step lies inside K
  const bool inside = wide_a && wide_w && m0 + TM <= M && n0 + TN <= N;
  auto fetch = [&](int k0) {
    if (inside && k0 + TK <= K) {
#pragma unroll
      for (int i = 0; i < GA; ++i) {
        const int gi = tid + i * GEMM_THREADS, row = gi / (TK / 4), k = k0 + (gi % (TK / 4)) * 4;
        load4<TA>(ra[i], A + (int64_t)(m0 + row) * lda + k, 4, true);
      }
#pragma unroll
      for (int i = 0; i < GW; ++i) {
        const int gi = tid + i * GEMM_THREADS, row = gi / (TK / 4), k = k0 + (gi % (TK / 4)) * 4;
        load4<TW>(rw[i], W + (int64_t)(n0 + row) * K + k, 4, true);
      }
      return;
    }
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
#pragma unroll
    for (int k = 0; k < TK; k += 2) {
      float a[BM], w[BN];
#pragma unroll
      for (int i = 0; i < BM; ++i) a[i] = a_s[k + half][wm + i * 32 + l32];
#pragma unroll
      for (int j = 0; j < BN; ++j) w[j] = w_s[k + half][wn + j * 32 + l32];
#pragma unroll
      for (int i = 0; i < BM; ++i)
#pragma unroll
        for (int j = 0; j < BN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], w[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < BM; ++i)
#pragma unroll
    for (int j = 0; j < BN; ++j) {
      const int n = n0 + wn + j * 32 + l32;
      if (n >= N) continue;
      const float b = bias ? Num<TW>::ld(bias + n) : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + i * 32 + half * 4 + 8 * (r / 4) + (r % 4);
        if (m >= M) continue;
        float v = acc[i][j][r];
        if (bias) v += b;
        Num<TC>::st(C + (int64_t)m * ldc + n, v);
      }
    }
}

// Up to 16 rows (a decode step): one wavefront per 16 columns, no LDS.  v_mfma_f32_16x16x4_f32 takes, from lane l, row
// l % 16 of A and of W at k = step + l / 16, and adds its four products into the accumulator in ascending k as fused
// multiply-adds (the same measurement as above): the bits of the other two kernels again.  A lane loads four
// consecutive elements of its row (16 bytes; the four lanes of a row 64 consecutive bytes), which is the operand of
// four steps once the four lanes of the row have exchanged elements (a 4 x 4 transpose in two rounds of swaps between
// lanes 16 and 32 apart).  Of FEW_SETS sets of FEW_DEPTH such loads of A and of W one is multiplied while the others
// are under way.
// Register r of lane l receives row 4 (l / 16) + r, column l % 16.
typedef __attribute__((ext_vector_type(4))) float f32x4;
#define FEW_DEPTH 8
#define FEW_SETS 2
#define FEW_DEPTH_BLOCKS 4     // ... with several blocks of rows (measured: 2, 4, 8)

// x[c] of the lane 16 s + i (s = 0..3) becomes what was x[s] of the lane 16 c + i: a 4 x 4 transpose between the
// registers and the wavefront's four rows of 16 lanes, by gfx950's row swaps (v_permlane16_swap exchanges the odd rows
// of its first operand with the even rows of its second, v_permlane32_swap the upper half of the first with the lower
// half of the second): the 2 x 2 blocks transposed in themselves, then the two off the diagonal exchanged
__device__ __forceinline__ void swap_rows_16(float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void swap_rows_32(float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void transpose_over_lane_rows(float (&x)[4]) {
  swap_rows_16(x[0], x[1]);
  swap_rows_16(x[2], x[3]);
  swap_rows_32(x[0], x[2]);
  swap_rows_32(x[1], x[3]);
}

// four consecutive elements at an address that is a multiple of four elements, no questions asked
template <typename T>
__device__ __forceinline__ void load4_aligned(float (&v)[4], const T* p) {
  load4<T>(v, p, 4, true);
}

template <typename TA, typename TW, typename TC, int RB>
__global__ __launch_bounds__(64) void gemm_nt_few_rows_kernel(TC* __restrict__ C, int64_t ldc,
                                                              const TA* __restrict__ A, int64_t lda,
                                                              const TW* __restrict__ W,
                                                              const TW* __restrict__ bias, int M, int N, int K,
                                                              int wide_a, int wide_w) {
  // RB blocks of 16 rows: the wavefront's 16 columns of W are loaded once for all of them, and the blocks' chains of
  // matrix instructions run side by side
  const int lane = threadIdx.x, i = lane & 15, kq = lane >> 4;
  const int n = blockIdx.x * 16 + i;
  const bool w_ok = n < N;
  // a lane whose row does not exist reads row 0 and drops what it read: no branch in the loop
  const TA* pa[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) pa[rb] = A + (int64_t)(16 * rb + i < M ? 16 * rb + i : 0) * lda + 4 * kq;
  const TW* pw = W + (int64_t)(w_ok ? n : 0) * K + 4 * kq;
  f32x4 acc[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
  // FEW_SETS sets of DEPTH loads of A's blocks and of W: one is multiplied while the others are on their way (a
  // wavefront has the registers of its SIMD to itself: so few wavefronts run here that the bytes each keeps under way
  // are what decides)
  constexpr int DEPTH = RB == 1 ? FEW_DEPTH : FEW_DEPTH_BLOCKS;
  float a[FEW_SETS][DEPTH][RB][4], w[FEW_SETS][DEPTH][4];
  // whole chunks of 16 elements, with aligned rows, take the loop without branches; what is left of K (and everything,
  // with rows that are not aligned) takes the careful loads afterwards: ascending k all the same
  const int chunks = (wide_a && wide_w) ? K / 16 : 0;
  // (a lane without a row of its own multiplies row 0's numbers: they meet nobody else's, a row of A and a row of W
  // make one element of C, and that element is not stored)
  auto multiply = [&](float (&x)[RB][4], float (&y)[4]) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) transpose_over_lane_rows(x[rb]);
    transpose_over_lane_rows(y);
#pragma unroll
    for (int st = 0; st < 4; ++st)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) acc[rb] = __builtin_amdgcn_mfma_f32_16x16x4f32(x[rb][st], y[st], acc[rb], 0, 0, 0);
  };
  // the loads of the chunks first .. first + DEPTH - 1 (those of them that exist; `all`: they all do)
  auto fetch = [&](float (&x)[DEPTH][RB][4], float (&y)[DEPTH][4], int first, bool all) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (all || first + d < chunks) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) load4_aligned<TA>(x[d][rb], pa[rb] + (first + d) * 16);
        load4_aligned<TW>(y[d], pw + (first + d) * 16);
      }
  };
  auto multiply_set = [&](float (&x)[DEPTH][RB][4], float (&y)[DEPTH][4], int first, bool all) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (all || first + d < chunks) multiply(x[d], y[d]);
  };
#pragma unroll
  for (int st = 0; st < FEW_SETS - 1; ++st) fetch(a[st], w[st], st * DEPTH, false);
  int c0 = 0;
  // while every set of a round and the sets asked for in it lie inside K nothing in the loop is conditional: the
  // compiler then counts the loads and waits for just those of the set it multiplies
  for (; c0 + (2 * FEW_SETS - 1) * DEPTH <= chunks; c0 += FEW_SETS * DEPTH) {
#pragma unroll
    for (int st = 0; st < FEW_SETS; ++st) {
      fetch(a[(st + FEW_SETS - 1) % FEW_SETS], w[(st + FEW_SETS - 1) % FEW_SETS], c0 + (st + FEW_SETS - 1) * DEPTH, true);
      multiply_set(a[st], w[st], c0 + st * DEPTH, true);
    }
  }
  for (; c0 < chunks; c0 += FEW_SETS * DEPTH) {
#pragma unroll
    for (int st = 0; st < FEW_SETS; ++st) {
      fetch(a[(st + FEW_SETS - 1) % FEW_SETS], w[(st + FEW_SETS - 1) % FEW_SETS], c0 + (st + FEW_SETS - 1) * DEPTH, false);
      multiply_set(a[st], w[st], c0 + st * DEPTH, false);
    }
  }
  for (int k0 = chunks * 16; k0 < K; k0 += 16) {
    const int k = k0 + 4 * kq;
    const int valid = k < K ? (K - k < 4 ? K - k : 4) : 0;
    float x[RB][4], y[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) x[rb][0] = x[rb][1] = x[rb][2] = x[rb][3] = 0.f;
    if (valid) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) load4<TA>(x[rb], pa[rb] + k0, valid, false);
      load4<TW>(y, pw + k0, valid, false);
    }
    multiply(x, y);
  }
  if (!w_ok) return;
  const float b = bias ? Num<TW>::ld(bias + n) : 0.f;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = 16 * rb + 4 * kq + r;
      if (m >= M) continue;
      float v = acc[rb][r];
      if (bias) v += b;
      Num<TC>::st(C + (int64_t)m * ldc + n, v);
    }
}

// in_bf16: A, W and bias are bfloat16 (else float); out_bf16: C is bfloat16 (else float).
extern "C" int ga_gemm_nt(void* C, int64_t ldc, const void* A, int64_t lda, const void* W,
                          const void* bias, int M, int N, int K, int in_bf16, int out_bf16,
                          hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return -1;
  // up to 64 rows: a wavefront per 16 columns, which it streams once for up to four blocks of 16 rows (with more than 32
  // rows and very many columns, a head over a large vocabulary, the plain kernel is faster: measured at 151,936 columns)
  const bool few = M <= GEMM_MATRIX_FROM_ROWS && !(M > 32 && N >= 65536);
  const int row_blocks = (M + 15) / 16;
  // many rows: the matrix cores, in the largest of the tiles 128 x 128, 128 x 64, 64 x 64 that still makes 256 workgroups
  const bool matrix = M > GEMM_MATRIX_FROM_ROWS;
  const bool wide = matrix && (int64_t)((M + 127) / 128) * ((N + 127) / 128) >= 256;
  const bool tall = matrix && !wide && (int64_t)((M + 127) / 128) * ((N + 63) / 64) >= 256;
  const int tm = (wide || tall) ? 128 : 64, tn = few ? 16 : wide ? 128 : 64;
  dim3 grid((N + tn - 1) / tn, (M + tm - 1) / tm), block(GEMM_THREADS);
  if (grid.y > 65535) return -2;
  // 16-byte loads (8 bytes for bfloat16) need rows that start at multiples of four elements
  const size_t unit = in_bf16 ? 8 : 16;
  const int wide_a = (K % 4 == 0 && lda % 4 == 0 && (uintptr_t)A % unit == 0) ? 1 : 0;
  const int wide_w = (K % 4 == 0 && (uintptr_t)W % unit == 0) ? 1 : 0;
#define LAUNCH(TA, TW, TC)                                                                                   \
  do {                                                                                                       \
    if (few && row_blocks == 1)                                                                              \
      hipLaunchKernelGGL((gemm_nt_few_rows_kernel<TA, TW, TC, 1>), grid, dim3(64), 0, stream, (TC*)C, ldc,   \
                         (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a, wide_w);         \
    else if (few && row_blocks == 2)                                                                         \
      hipLaunchKernelGGL((gemm_nt_few_rows_kernel<TA, TW, TC, 2>), grid, dim3(64), 0, stream, (TC*)C, ldc,   \
                         (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a, wide_w);         \
    else if (few && row_blocks == 3)                                                                         \
      hipLaunchKernelGGL((gemm_nt_few_rows_kernel<TA, TW, TC, 3>), grid, dim3(64), 0, stream, (TC*)C, ldc,   \
                         (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a, wide_w);         \
    else if (few)                                                                                            \
      hipLaunchKernelGGL((gemm_nt_few_rows_kernel<TA, TW, TC, 4>), grid, dim3(64), 0, stream, (TC*)C, ldc,   \
                         (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a, wide_w);         \
    else if (matrix && wide)                                                                                 \
      hipLaunchKernelGGL((gemm_nt_matrix_kernel<TA, TW, TC, 128, 128, 32>), grid, block, 0, stream,          \
                         (TC*)C, ldc, (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a,     \
                         wide_w);                                                                            \
    else if (matrix && tall)                                                                                 \
      hipLaunchKernelGGL((gemm_nt_matrix_kernel<TA, TW, TC, 128, 64, 32>), grid, block, 0, stream,           \
                         (TC*)C, ldc, (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a,     \
                         wide_w);                                                                            \
    else if (matrix)                                                                                         \
      hipLaunchKernelGGL((gemm_nt_matrix_kernel<TA, TW, TC, 64, 64, 32>), grid, block, 0, stream,            \
                         (TC*)C, ldc, (const TA*)A, lda, (const TW*)W, (const TW*)bias, M, N, K, wide_a,     \
                         wide_w);                                                                            \
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
