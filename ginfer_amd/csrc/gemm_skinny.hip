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

// A root-mean-square norm folded into the two products around it (ginfer/core/op/kernels/cuda/rmsnorm_kernel.cu:27-66
// is the norm itself: y = x * g / sqrtf(sum(x^2) / width + eps)).  The product BEFORE the norm adds its result
// to the 32-bit residual stream, writes h * g rounded once, and one partial sum of h^2 per row and workgroup
// (NormOut).  The product AFTER it runs on h * g and multiplies every sum by 1 / sqrtf(sum / width + eps), the
// partial sums added in a fixed order (NormIn): the same value as normalising first, without the norm's own
// pass over memory.  At most 16 rows.
struct NormIn {
  const float* sumsq;      // [M][parts], or null: the rows are used as they are
  int parts;
  float inv_width, eps;
};
struct NormOut {
  float* residual;         // [M][N] (row stride ldr), read and written; null: a plain product
  int64_t ldr;
  const void* gain;        // [N], bfloat16 or float
  int gain_f32;
  bf16_t* scaled;          // [M][N] (row stride lds): (residual + product) * gain
  int64_t lds;
  float* sumsq;            // [M][gridDim.x]
};
#define NORM_IN_EARLY 2    // partial sums per row a lane asks for ahead of time: 128 parts, a width of 2048
#define NORM_IN_MAX_PARTS 512

// Partial sums of the rows' squares: wavefront w takes rows 2w and 2w + 1 of the 16.  The first 128 parts of a
// row are asked for at the start of a kernel, so that they arrive while the weights stream (more would cost
// the registers that the weights' loads need); any further ones are fetched at the end.
struct NormInLoads {
  float v[2][NORM_IN_EARLY];
  __device__ __forceinline__ void load(const NormIn& in, int M, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NORM_IN_EARLY; ++j) {
        const int m = wave * 2 + i, p = lane + 64 * j;
        v[i][j] = (in.sumsq && m < M && p < in.parts) ? in.sumsq[(int64_t)m * in.parts + p] : 0.f;
      }
  }
  // the rows' factors; rstd: 16 floats of LDS, a barrier before they are read.  Lane l adds parts l, l + 64, ...
  // in ascending order, then the lanes add up in a butterfly: the order never depends on the data.
  __device__ __forceinline__ void finish(const NormIn& in, float* rstd, int M, int wave, int lane) const {
    if (!in.sumsq) return;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = wave * 2 + i;
      float t = 0.f;
#pragma unroll
      for (int j = 0; j < NORM_IN_EARLY; ++j) t += v[i][j];
      if (m < M)
        for (int p = lane + 64 * NORM_IN_EARLY; p < in.parts; p += 64) t += in.sumsq[(int64_t)m * in.parts + p];
      t = wave_sum(t);
      if (lane == 0) rstd[m] = 1.0f / sqrtf(t * in.inv_width + in.eps);
    }
  }
};

// The wavefront's share of the sum over k in [kb, ke): UNROLL steps of 64 elements per trip, all loads of a
// trip issued before its products.  The guard on every 8-element piece makes the tail of the range safe
// (a piece past the end is zeros and touches no memory); the terms are added in ascending k.
template <int NT, int MB, int UNROLL>
struct SkinnyTrip {
  bf16x8 a[UNROLL][2][NT], b[UNROLL][2][MB];
  __device__ __forceinline__ void load(const bf16_t* const (&wp)[NT], const bool (&wok)[NT],
                                       const bf16_t* const (&ap)[MB], const bool (&aok)[MB], int k, int ke, int g) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int kk = k + u * 64 + g * 16 + j * 8;
        const bool ok = kk < ke;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) a[u][j][nt] = (ok && wok[nt]) ? load8(wp[nt] + kk) : zero8();
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) b[u][j][mb] = (ok && aok[mb]) ? load8(ap[mb] + kk) : zero8();
      }
  }
  __device__ __forceinline__ void multiply(f32x4 (&acc)[NT][MB]) const {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[nt][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][j][nt], b[u][j][mb], acc[nt][mb], 0, 0, 0);
  }
};

template <int NT, int MB>
__device__ __forceinline__ void skinny_accumulate(f32x4 (&acc)[NT][MB], const bf16_t* const (&wp)[NT],
                                                  const bool (&wok)[NT], const bf16_t* const (&ap)[MB],
                                                  const bool (&aok)[MB], int kb, int ke, int g) {
  constexpr int UNROLL = (NT * MB <= 4) ? 4 : 2;
  for (int k = kb; k < ke; k += 64 * UNROLL) {
    SkinnyTrip<NT, MB, UNROLL> trip;
    trip.load(wp, wok, ap, aok, k, ke, g);
    trip.multiply(acc);
  }
}

// NT: 16-row tiles of W per wavefront; MB: 16-row blocks of A; KS: wavefronts of a workgroup that split K
// for the same rows (the workgroup's SK_WAVES / KS groups own different rows of W).  The grid's y
// dimension splits K further: then every workgroup writes its part in 32-bit to P[y][M][N] and the
// consumer adds the parts in order (the bias rides on part 0).
// GATED (NT == 2): W holds two stacked matrices of N rows each (gate over up); the wavefront's two tiles
// are rows n0.. of the gate and the same rows of the up matrix, and the epilogue writes
// silu(gate) * up = (g * (1 / (1 + exp(-g)))) * u (ginfer/core/op/kernels/cuda/swiglu_kernel.cu:24-27) for N
// columns: the activation of the feed-forward without a pass over memory of its own.
template <int NT, int MB, int KS, typename TC, bool GATED>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(TC* __restrict__ C, int64_t ldc,
                                                                 const bf16_t* __restrict__ A, int64_t lda,
                                                                 const bf16_t* __restrict__ W,
                                                                 const bf16_t* __restrict__ bias, int M, int N,
                                                                 int K, int kchunk_wg, int kchunk_wave,
                                                                 NormIn norm_in, NormOut norm_out) {
  __shared__ float red[SK_WAVES][NT * 16][MB * 16 + 1];
  __shared__ float rstd[16];
  constexpr int GROUPS = SK_WAVES / KS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int grp = wave / KS, ks = wave % KS;
  constexpr int NCOL = GATED ? 16 : NT * 16;       // output columns of a group
  const int n0 = (blockIdx.x * GROUPS + grp) * NCOL;
  const int kwg = blockIdx.y * kchunk_wg;
  const int kwg_end = kwg + kchunk_wg < K ? kwg + kchunk_wg : K;
  const int kb = kwg + ks * kchunk_wave;
  const int ke = kb + kchunk_wave < kwg_end ? kb + kchunk_wave : kwg_end;

  const bf16_t* wp[NT];
  bool wok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = GATED ? n0 + r : n0 + nt * 16 + r;
    wok[nt] = n < N;
    wp[nt] = W + ((int64_t)(wok[nt] ? n : 0) + (GATED ? (int64_t)nt * N : 0)) * K;
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
  // what the epilogue needs from memory is asked for now, so that it arrives while the weights stream
  NormInLoads in_loads;
  if (MB == 1) in_loads.load(norm_in, M, wave, lane);
  float out_res = 0.f, out_gain = 0.f;       // NormOut: thread t holds row t / 16, column t % 16 of the workgroup
  const bool fuse_out = !GATED && NT == 1 && KS == SK_WAVES && MB == 1 && norm_out.residual != nullptr;
  if (fuse_out) {
    const int m = threadIdx.x / 16, n = blockIdx.x * 16 + threadIdx.x % 16;
    if (threadIdx.x < 256 && m < M && n < N) {
      out_res = norm_out.residual[(int64_t)m * norm_out.ldr + n];
      out_gain = norm_out.gain_f32 ? reinterpret_cast<const float*>(norm_out.gain)[n]
                                   : bf16_to_f32(reinterpret_cast<const bf16_t*>(norm_out.gain)[n]);
    }
  }

  skinny_accumulate<NT, MB>(acc, wp, wok, ap, aok, kb, ke, g);
  if (MB == 1) in_loads.finish(norm_in, rstd, M, wave, lane);
  // the KS parts of a group meet in LDS and are added in wavefront order
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][nt * 16 + g * 4 + i][mb * 16 + r] = acc[nt][mb][i];
  __syncthreads();
  const bool scale_rows = MB == 1 && norm_in.sumsq != nullptr;
  if (fuse_out) {
    // 16 columns of 16 rows: the threads of a row are 16 neighbouring lanes, which add up their squares
    if (threadIdx.x >= 256) return;
    const int nl = threadIdx.x % 16, m = threadIdx.x / 16, n = blockIdx.x * 16 + nl;
    const bool ok = m < M && n < N;
    float h = 0.f;
    if (ok) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < KS; ++w) v += red[w][nl][m];
      if (scale_rows) v *= rstd[m];
      if (bias) v += bf16_to_f32(bias[n]);
      h = out_res + v;
      norm_out.residual[(int64_t)m * norm_out.ldr + n] = h;
      norm_out.scaled[(int64_t)m * norm_out.lds + n] = f32_to_bf16(h * out_gain);
    }
    float sq = h * h;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, WAVE);
    if (nl == 0 && m < M) norm_out.sumsq[(int64_t)m * gridDim.x + blockIdx.x] = sq;
    return;
  }
  const bool partial = gridDim.y > 1;
  float* P = reinterpret_cast<float*>(C) + (int64_t)blockIdx.y * M * N;      // parts are [y][M][N], dense
  for (int idx = threadIdx.x; idx < GROUPS * NCOL * MB * 16; idx += SK_THREADS) {
    const int nl = idx % NCOL, rest = idx / NCOL;
    const int gi = rest % GROUPS, m = rest / GROUPS;
    const int n = (blockIdx.x * GROUPS + gi) * NCOL + nl;
    if (m >= M || n >= N) continue;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < KS; ++w) v += red[gi * KS + w][nl][m];
    if (scale_rows) v *= rstd[m];
    if (GATED) {
      float u = 0.f;
#pragma unroll
      for (int w = 0; w < KS; ++w) u += red[gi * KS + w][16 + nl][m];
      if (scale_rows) u *= rstd[m];
      v = (v * (1.0f / (1.0f + expf(-v)))) * u;
    }
    if (bias && blockIdx.y == 0) v += bf16_to_f32(bias[n]);
    if (partial) P[(int64_t)m * N + n] = v;
    else Num<TC>::st(C + (int64_t)m * ldc + n, v);
  }
}

// What ga_gemm_skinny takes beside the product itself; all null or zero for a plain product.
struct GaSkinnyNorm {
  const float* in_sumsq;   // [M][in_parts]: the rows of A are (h * g) of a norm whose sums these are
  int in_parts;
  float inv_width, eps;
  float* residual;         // [M][N], row stride ldr: the product is added to it (C is not written)
  int64_t ldr;
  const void* gain;        // [N] of the norm that follows
  int gain_f32;
  void* scaled;            // bfloat16 [M][N], row stride lds
  int64_t lds;
  float* out_sumsq;        // [M][ga_skinny_norm_parts(N)]
};

// Partial sums a row gets from a product with N columns that feeds a norm.
extern "C" int ga_skinny_norm_parts(int N) { return (N + 15) / 16; }

// A [M, K] (row stride lda), W [N, K] contiguous, bias [N] or null.  grid_splits == 1: C [M, N] (row
// stride ldc) in bfloat16 or float.  grid_splits > 1: C is float [grid_splits][M][N], parts to be added
// by the consumer.  gated: W is [2N, K] (gate over up), C [M, N] = silu(A.gate^T) * (A.up^T), no bias, no
// grid split.  M <= 64, K a multiple of 8, rows 16-byte aligned.  nt in {1,2,4}, ks in {1,2,4,8}; 0 lets
// the library choose.
extern "C" int ga_gemm_skinny(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias,
                              int M, int N, int K, int out_f32, int nt, int ks, int grid_splits, int gated,
                              const GaSkinnyNorm* norm, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 || lda % 8 || grid_splits < 1) return -1;
  const int mb = (M + 15) / 16;
  NormIn norm_in = {nullptr, 0, 0.f, 0.f};
  NormOut norm_out = {nullptr, 0, nullptr, 0, nullptr, 0, nullptr};
  if (norm && norm->in_sumsq) {
    if (mb != 1 || norm->in_parts < 1 || norm->in_parts > NORM_IN_MAX_PARTS) return -5;
    norm_in = NormIn{norm->in_sumsq, norm->in_parts, norm->inv_width, norm->eps};
  }
  if (norm && norm->residual) {
    if (mb != 1 || gated || grid_splits != 1 || !norm->gain || !norm->scaled || !norm->out_sumsq) return -6;
    nt = 1;
    ks = SK_WAVES;
    norm_out = NormOut{norm->residual, norm->ldr, norm->gain, norm->gain_f32, (bf16_t*)norm->scaled, norm->lds,
                       norm->out_sumsq};
  }
  if (gated) nt = 2;
  if (nt == 0) nt = (N >= 4096 && mb > 1) ? 4 : 1;
  if (ks == 0) ks = 8;
  if ((nt != 1 && nt != 2 && nt != 4) || (ks != 1 && ks != 2 && ks != 4 && ks != 8)) return -2;
  if (nt == 4 && mb > 2 && ks < 2) return -2;      // LDS of the reduction
  if (grid_splits > 1 && !out_f32) return -3;
  if (gated && (grid_splits > 1 || bias)) return -4;
  const int groups = SK_WAVES / ks;
  const int ncol = gated ? 16 : nt * 16;
  const int kchunk_wg = ((K + grid_splits - 1) / grid_splits + 63) / 64 * 64;
  const int kchunk_wave = ((kchunk_wg + ks - 1) / ks + 63) / 64 * 64;
  dim3 grid((N + groups * ncol - 1) / (groups * ncol), grid_splits), block(SK_THREADS);
#define LAUNCH(NT, MB, KS, TC, G)                                                                       \
  hipLaunchKernelGGL((gemm_skinny_kernel<NT, MB, KS, TC, G>), grid, block, 0, stream, (TC*)C, ldc,     \
                     (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, M, N, K, kchunk_wg, \
                     kchunk_wave, norm_in, norm_out)
#define PICK_KS(NT, MB, TC, G)                                                                          \
  switch (ks) {                                                                                         \
    case 1: LAUNCH(NT, MB, 1, TC, G); break;                                                            \
    case 2: LAUNCH(NT, MB, 2, TC, G); break;                                                            \
    case 4: LAUNCH(NT, MB, 4, TC, G); break;                                                            \
    default: LAUNCH(NT, MB, 8, TC, G); break;                                                           \
  }
#define PICK_MB(NT, TC, G)                                                                              \
  switch (mb) {                                                                                         \
    case 1: PICK_KS(NT, 1, TC, G) break;                                                                \
    case 2: PICK_KS(NT, 2, TC, G) break;                                                                \
    case 3: PICK_KS(NT, 3, TC, G) break;                                                                \
    default: PICK_KS(NT, 4, TC, G) break;                                                               \
  }
#define PICK_NT(TC)                                                                                     \
  switch (nt) {                                                                                         \
    case 1: PICK_MB(1, TC, false) break;                                                                \
    case 2: PICK_MB(2, TC, false) break;                                                                \
    default: PICK_MB(4, TC, false) break;                                                               \
  }
  if (gated) {
    if (out_f32) { PICK_MB(2, float, true) } else { PICK_MB(2, bf16_t, true) }
  } else if (out_f32) {
    PICK_NT(float)
  } else {
    PICK_NT(bf16_t)
  }
#undef PICK_NT
#undef PICK_MB
#undef PICK_KS
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}

// The fused q|k|v projection of a decode step with its epilogue: bias, NeoX rotation of q and k
// (ginfer/core/op/kernels/cuda/rope_kernel.cu:83-102, on the 32-bit sums: one rounding fewer than rotating
// the rounded projection), q to its own buffer, k and v straight into the paged cache (v transposed;
// ginfer/core/op/kernels/cuda/store_kvcache_kernel.cu:19-30).  A wavefront group owns a UNIT of 32 output
// columns as two tiles of 16: for a q or k head the columns j0..j0+15 and their rotation partners
// j0+half..; for a v head 32 consecutive columns.  head_dim a multiple of 32, rotary_dim == head_dim.
template <int MB, int KS>
__global__ __launch_bounds__(SK_THREADS) void qkv_rope_skinny_kernel(
    bf16_t* __restrict__ q_out, const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W,
    const bf16_t* __restrict__ bias, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int64_t* __restrict__ slot_mapping, bf16_t* __restrict__ k_pages,
    bf16_t* __restrict__ v_pages, int M, int K, int nh, int nkv, int hd, int page_size, int write_kv,
    int kchunk_wave, NormIn norm_in) {
  __shared__ float red[SK_WAVES][32][MB * 16 + 1];
  __shared__ float rstd[16];
  constexpr int GROUPS = SK_WAVES / KS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int grp = wave / KS, ks = wave % KS;
  const int half = hd >> 1, upq = half / 16;            // units per q or k head
  const int qk_units = (nh + nkv) * upq, units = qk_units + nkv * (hd / 32);
  const int unit = blockIdx.x * GROUPS + grp;
  const bool unit_ok = unit < units;
  // first rows of the unit's two tiles
  int row0 = 0, row1 = 0;
  if (unit_ok) {
    if (unit < qk_units) {
      row0 = (unit / upq) * hd + (unit % upq) * 16;
      row1 = row0 + half;
    } else {
      const int u = unit - qk_units;
      row0 = (nh + nkv) * hd + u * 32;
      row1 = row0 + 16;
    }
  }
  const int kb = ks * kchunk_wave;
  const int ke = kb + kchunk_wave < K ? kb + kchunk_wave : K;
  const bf16_t* wp[2] = {W + (int64_t)(row0 + r) * K, W + (int64_t)(row1 + r) * K};
  const bool wok[2] = {unit_ok, unit_ok};
  const bf16_t* ap[MB];
  bool aok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + r;
    aok[mb] = m < M;
    ap[mb] = A + (int64_t)(aok[mb] ? m : 0) * lda;
  }
  // What the epilogue needs from memory (position, slot, cosine and sine, bias) is asked for now, so that
  // it arrives while the weights stream: an epilogue item is (unit of the workgroup, column, row of A).
  constexpr int ITEMS = (GROUPS * 16 * MB * 16 + SK_THREADS - 1) / SK_THREADS;
  int64_t e_slot[ITEMS];
  float e_cos[ITEMS], e_sin[ITEMS], e_blo[ITEMS], e_bhi[ITEMS];
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int idx = threadIdx.x + it * SK_THREADS;
    const int nl = idx % 16, rest = idx / 16;
    const int gi = rest % GROUPS, m = rest / GROUPS;
    const int u = blockIdx.x * GROUPS + gi;
    e_slot[it] = -1;
    e_cos[it] = 1.f;
    e_sin[it] = e_blo[it] = e_bhi[it] = 0.f;
    if (m < M && u < units) {
      if (write_kv) e_slot[it] = slot_mapping[m];
      if (u < qk_units) {
        const int head = u / upq, j = (u % upq) * 16 + nl;
        const int p = positions[m];
        e_cos[it] = cos_t[(int64_t)p * half + j];
        e_sin[it] = sin_t[(int64_t)p * half + j];
        if (bias) {
          e_blo[it] = bf16_to_f32(bias[head * hd + j]);
          e_bhi[it] = bf16_to_f32(bias[head * hd + j + half]);
        }
      } else if (bias) {
        const int v = u - qk_units;
        const int at = (nh + nkv + v / (hd / 32)) * hd + (v % (hd / 32)) * 32 + nl;
        e_blo[it] = bf16_to_f32(bias[at]);
        e_bhi[it] = bf16_to_f32(bias[at + 16]);
      }
    }
  }
  f32x4 acc[2][MB];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  NormInLoads in_loads;
  if (MB == 1) in_loads.load(norm_in, M, wave, lane);
  skinny_accumulate<2, MB>(acc, wp, wok, ap, aok, kb, ke, g);
  if (MB == 1) in_loads.finish(norm_in, rstd, M, wave, lane);
  const bool scale_rows = MB == 1 && norm_in.sumsq != nullptr;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][nt * 16 + g * 4 + i][mb * 16 + r] = acc[nt][mb][i];
  __syncthreads();
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int idx = threadIdx.x + it * SK_THREADS;
    const int nl = idx % 16, rest = idx / 16;
    const int gi = rest % GROUPS, m = rest / GROUPS;
    const int u = blockIdx.x * GROUPS + gi;
    if (m >= M || u >= units) continue;
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int w = 0; w < KS; ++w) {
      lo += red[gi * KS + w][nl][m];
      hi += red[gi * KS + w][16 + nl][m];
    }
    if (scale_rows) {
      lo *= rstd[m];
      hi *= rstd[m];
    }
    lo += e_blo[it];
    hi += e_bhi[it];
    const int64_t slot = e_slot[it];
    const int64_t page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot - page * page_size : 0;
    if (u < qk_units) {
      const int head = u / upq, j = (u % upq) * 16 + nl;
      const float c = e_cos[it], sn = e_sin[it];
      const bf16_t olo = f32_to_bf16(lo * c - hi * sn), ohi = f32_to_bf16(lo * sn + hi * c);
      if (head < nh) {
        bf16_t* o = q_out + (int64_t)m * nh * hd + (int64_t)head * hd + j;
        o[0] = olo;
        o[half] = ohi;
      } else if (slot >= 0) {
        bf16_t* o = k_pages + ((page * nkv + (head - nh)) * page_size + off) * hd + j;
        o[0] = olo;
        o[half] = ohi;
      }
    } else if (slot >= 0) {
      const int v = u - qk_units;
      const int gh = v / (hd / 32), d = (v % (hd / 32)) * 32 + nl;
      bf16_t* o = v_pages + ((page * nkv + gh) * (int64_t)hd + d) * page_size + off;
      o[0] = f32_to_bf16(lo);
      o[(int64_t)16 * page_size] = f32_to_bf16(hi);
    }
  }
}

// q_out [M, nh*hd]; A [M, K] (row stride lda); W [(nh + 2 nkv) hd, K]; bias [(nh + 2 nkv) hd] or null;
// positions int32 [M]; cos_t, sin_t float [positions, hd/2]; slot_mapping int64 [M] (-1: no cache write);
// k_pages [pages, nkv, page_size, hd], v_pages [pages, nkv, hd, page_size].  norm: null, or the sums of the
// norm whose (h * g) the rows of A are (its in_ fields only).
extern "C" int ga_qkv_rope_skinny(void* q_out, const void* A, int64_t lda, const void* W, const void* bias,
                                  const void* positions, const void* cos_t, const void* sin_t,
                                  const void* slot_mapping, void* k_pages, void* v_pages, int M, int K, int nh,
                                  int nkv, int hd, int page_size, int write_kv, const GaSkinnyNorm* norm,
                                  hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 || lda % 8 || hd % 32 || nh <= 0 || nkv <= 0) return -1;
  const int mb = (M + 15) / 16;
  NormIn norm_in = {nullptr, 0, 0.f, 0.f};
  if (norm && norm->residual) return -6;
  if (norm && norm->in_sumsq) {
    if (mb != 1 || norm->in_parts < 1 || norm->in_parts > NORM_IN_MAX_PARTS) return -5;
    norm_in = NormIn{norm->in_sumsq, norm->in_parts, norm->inv_width, norm->eps};
  }
  const int ks = 8, groups = SK_WAVES / ks;
  const int units = (nh + 2 * nkv) * hd / 32;
  const int kchunk_wave = ((K + ks - 1) / ks + 63) / 64 * 64;
  dim3 grid((units + groups - 1) / groups), block(SK_THREADS);
#define LAUNCH(MB)                                                                                        \
  hipLaunchKernelGGL((qkv_rope_skinny_kernel<MB, 8>), grid, block, 0, stream, (bf16_t*)q_out,            \
                     (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, (const int32_t*)positions, \
                     (const float*)cos_t, (const float*)sin_t, (const int64_t*)slot_mapping, (bf16_t*)k_pages, \
                     (bf16_t*)v_pages, M, K, nh, nkv, hd, page_size, write_kv, kchunk_wave, norm_in)
  switch (mb) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 3: LAUNCH(3); break;
    default: LAUNCH(4); break;
  }
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
