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
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

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
#define NORM_IN_MAX_PARTS 512

// Partial sums of the rows' squares.  With up to 8 rows wavefront w takes row w, else rows 2w and 2w + 1.  Four
// values per lane are asked for at the start of a kernel, so that they arrive while the weights stream (more
// would cost the registers that the weights' loads need): 256 parts of a row, or 128 of each of two; any
// further ones are fetched at the end.
struct NormInLoads {
  float v[4];
  __device__ __forceinline__ void load(const NormIn& in, int M, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = M <= 8 ? wave : wave * 2 + (j >> 1);
      const int p = M <= 8 ? lane + 64 * j : lane + 64 * (j & 1);
      v[j] = (in.sumsq && m < M && p < in.parts) ? in.sumsq[(int64_t)m * in.parts + p] : 0.f;
    }
  }
  // the rows' factors; rstd: 16 floats of LDS, a barrier before they are read.  Lane l adds parts l, l + 64, ...
  // in ascending order, then the lanes add up in a butterfly: the order never depends on the data.
  __device__ __forceinline__ void finish(const NormIn& in, float* rstd, int M, int wave, int lane) const {
    if (!in.sumsq) return;
    const int rows = M <= 8 ? 1 : 2, early = M <= 8 ? 4 : 2;
    for (int i = 0; i < rows; ++i) {
      const int m = M <= 8 ? wave : wave * 2 + i;
      float t = M <= 8 ? (v[0] + v[1]) + (v[2] + v[3]) : (i == 0 ? v[0] + v[1] : v[2] + v[3]);
      if (m < M)
        for (int p = lane + 64 * early; p < in.parts; p += 64) t += in.sumsq[(int64_t)m * in.parts + p];
      t = wave_sum(t);
      if (lane == 0 && m < 16) rstd[m] = 1.0f / sqrtf(t * in.inv_width + in.eps);
    }
  }
};

// The wavefront's share of the sum over k: UNROLL steps of 64 elements per trip, all loads of a trip issued
// before its products.  The trips run over [kb, kend), the same for every lane; a lane's own pointers may be
// shifted (a packed tile, below) and its own range ends at ke: the guard on every 8-element piece makes the
// tail safe (a piece past the end is zeros and touches no memory).  The terms are added in ascending k.
template <int NT, int MB, int UNROLL>
struct SkinnyTrip {
  bf16x8 a[UNROLL][2][NT], b[UNROLL][2][MB];
  __device__ __forceinline__ void load(const bf16_t* const (&wp)[NT], const bool (&wok)[NT],
                                       const bf16_t* const (&ap)[MB], const bool (&aok)[MB], int k, int ke, int g) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int kk = k + u * 64 + j * 32 + g * 8;
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

template <int NT, int MB, int UNROLL = ((NT * MB <= 4) ? 4 : 2)>
__device__ __forceinline__ void skinny_accumulate(f32x4 (&acc)[NT][MB], const bf16_t* const (&wp)[NT],
                                                  const bool (&wok)[NT], const bf16_t* const (&ap)[MB],
                                                  const bool (&aok)[MB], int kb, int kend, int ke, int g) {
  for (int k = kb; k < kend; k += 64 * UNROLL) {
    SkinnyTrip<NT, MB, UNROLL> trip;
    trip.load(wp, wok, ap, aok, k, ke, g);
    trip.multiply(acc);
  }
}

// A PACKED tile (PACK == 2, at most 8 rows of A): with so few rows half of the matrix core's 16 x 16 tile
// would hold nothing, so the tile takes 8 rows of W twice, for the two halves of the wavefront's K range:
// tile row q * 8 + c is row c of W over half q, tile column q * 8 + m is row m of A over half q, and
// C[m][c] = D[c][m] + D[8 + c][8 + m] (the other entries mix the halves and are dropped).  A workgroup then
// owns half as many columns over the same K: twice the workgroups stream the weights, with every lane still
// loading, which is what a product with few columns lacks to fill the chip.
template <int PACK>
struct Packed {
  static constexpr int CP = 16 / PACK;     // columns of W in a tile = most rows of A
  // lane row r of a tile: its column of W (and row of A), and its half of K
  static __device__ __forceinline__ int col(int r) { return r % CP; }
  static __device__ __forceinline__ int seg(int r) { return r / CP; }
};

// How K is dealt out: in steps of 64 elements, as evenly as whole steps allow, to `units` consumers (the
// wavefronts that split K, over all workgroups of a column, times the halves of a packed tile).  Consumer u
// takes the steps [u * steps / units, (u + 1) * steps / units).  A lane works in its own coordinates, starting
// at 0 at its first element: `shift` is where that lies, `ke` its own end, `kend` the end of the wavefront's
// trips (the longer of its halves).
template <int PACK>
struct KRange {
  int shift, ke, kend;
  __device__ __forceinline__ KRange(int first_unit, int seg, int steps, int units, int K) {
    int longest = 0;
#pragma unroll
    for (int q = 0; q < PACK; ++q) {
      const int b = (int)(((int64_t)(first_unit + q) * steps) / units), e = (int)(((int64_t)(first_unit + q + 1) * steps) / units);
      longest = e - b > longest ? e - b : longest;
      if (q == seg) {
        shift = b * 64;
        ke = (e * 64 < K ? e * 64 : K) - b * 64;
      }
    }
    kend = longest * 64;
  }
};

// NT: tiles of W per wavefront; MB: 16-row blocks of A; KS: wavefronts of a workgroup that split K
// for the same rows (the workgroup's SK_WAVES / KS groups own different rows of W).  The grid's y
// dimension splits K further: then every workgroup writes its part in 32-bit to P[y][M][N] and the
// consumer adds the parts in order (the bias rides on part 0).
// GATED (NT == 2): W holds two stacked matrices of N rows each (gate over up); the wavefront's two tiles
// are rows n0.. of the gate and the same rows of the up matrix, and the epilogue writes
// silu(gate) * up = (g * (1 / (1 + exp(-g)))) * u (ginfer/core/op/kernels/cuda/swiglu_kernel.cu:24-27) for N
// columns: the activation of the feed-forward without a pass over memory of its own.
template <int NT, int MB, int KS, typename TC, bool GATED, int PACK>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(TC* __restrict__ C, int64_t ldc,
                                                                 const bf16_t* __restrict__ A, int64_t lda,
                                                                 const bf16_t* __restrict__ W,
                                                                 const bf16_t* __restrict__ bias, int M, int N,
                                                                 int K, int ksteps, NormIn norm_in,
                                                                 NormOut norm_out, int fold_cols) {
  static_assert(PACK == 1 || MB == 1, "a packed tile holds at most 8 rows of A");
  __shared__ float red[SK_WAVES][NT * 16][MB * 16 + 1];
  __shared__ float rstd[16];
  using P = Packed<PACK>;
  constexpr int CP = P::CP;
  constexpr int GROUPS = SK_WAVES / KS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int grp = wave / KS, ks = wave % KS;
  constexpr int NCOL = GATED ? CP : NT * CP;       // output columns of a group
  // A product that folds the norm after it owns `fold_cols` (<= CP) columns per workgroup: as many as spread the
  // columns over all compute units (every workgroup reads all rows of A, so fewer, larger workgroups cost more
  // than the empty tile rows of more, smaller ones).
  const bool fuse_out = !GATED && NT == 1 && KS == SK_WAVES && MB == 1 && norm_out.residual != nullptr;
  const int my_cols = fuse_out ? fold_cols : NCOL;
  const int n0 = fuse_out ? blockIdx.x * fold_cols : (blockIdx.x * GROUPS + grp) * NCOL;
  const KRange<PACK> kr((blockIdx.y * KS + ks) * PACK, P::seg(r), ksteps, gridDim.y * KS * PACK, K);
  const int shift = kr.shift;

  const bf16_t* wp[NT];
  bool wok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = GATED ? n0 + P::col(r) : n0 + nt * CP + P::col(r);
    wok[nt] = n < N && (!fuse_out || P::col(r) < my_cols);
    wp[nt] = W + ((int64_t)(wok[nt] ? n : 0) + (GATED ? (int64_t)nt * N : 0)) * K + shift;
  }
  const bf16_t* ap[MB];
  bool aok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + P::col(r);
    aok[mb] = m < M;
    ap[mb] = A + (int64_t)(aok[mb] ? m : 0) * lda + shift;
  }
  f32x4 acc[NT][MB];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  // what the epilogue needs from memory is asked for now, so that it arrives while the weights stream
  NormInLoads in_loads;
  if (MB == 1) in_loads.load(norm_in, M, wave, lane);
  float out_res = 0.f, out_gain = 0.f;       // NormOut: thread t holds row t / CP, column t % CP of the workgroup
  if (fuse_out) {
    const int m = threadIdx.x / CP, n = n0 + threadIdx.x % CP;
    if (threadIdx.x < CP * CP && m < M && n < N && threadIdx.x % CP < my_cols) {
      out_res = norm_out.residual[(int64_t)m * norm_out.ldr + n];
      out_gain = norm_out.gain_f32 ? reinterpret_cast<const float*>(norm_out.gain)[n]
                                   : bf16_to_f32(reinterpret_cast<const bf16_t*>(norm_out.gain)[n]);
    }
  }

  skinny_accumulate<NT, MB>(acc, wp, wok, ap, aok, 0, kr.kend, kr.ke, g);
  if (MB == 1) in_loads.finish(norm_in, rstd, M, wave, lane);
  // the KS parts of a group meet in LDS and are added in wavefront order, the halves of a packed tile in theirs
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][nt * 16 + g * 4 + i][mb * 16 + r] = acc[nt][mb][i];
  __syncthreads();
  const bool scale_rows = MB == 1 && norm_in.sumsq != nullptr;
  // element (column nl of tile t, row m) of group gi, summed over its wavefronts and halves
  auto total = [&](int gi, int t, int nl, int m) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < KS; ++w)
#pragma unroll
      for (int q = 0; q < PACK; ++q) v += red[gi * KS + w][t * 16 + q * CP + nl][(m / CP) * 16 + q * CP + m % CP];
    return v;
  };
  if (fuse_out) {
    // CP columns of up to CP rows: the threads of a row are CP neighbouring lanes, which add up their squares
    if (threadIdx.x >= CP * CP) return;
    const int nl = threadIdx.x % CP, m = threadIdx.x / CP, n = n0 + nl;
    const bool ok = m < M && n < N && nl < my_cols;
    float h = 0.f;
    if (ok) {
      float v = total(0, 0, nl, m);
      if (scale_rows) v *= rstd[m];
      if (bias) v += bf16_to_f32(bias[n]);
      h = out_res + v;
      norm_out.residual[(int64_t)m * norm_out.ldr + n] = h;
      norm_out.scaled[(int64_t)m * norm_out.lds + n] = f32_to_bf16(h * out_gain);
    }
    float sq = h * h;
#pragma unroll
    for (int o = CP / 2; o > 0; o >>= 1) sq += __shfl_xor(sq, o, WAVE);
    if (nl == 0 && m < M) norm_out.sumsq[(int64_t)m * gridDim.x + blockIdx.x] = sq;
    return;
  }
  const bool partial = gridDim.y > 1;
  float* Pp = reinterpret_cast<float*>(C) + (int64_t)blockIdx.y * M * N;      // parts are [y][M][N], dense
  constexpr int MROWS = PACK == 1 ? MB * 16 : CP;
  for (int idx = threadIdx.x; idx < GROUPS * NCOL * MROWS; idx += SK_THREADS) {
    const int nl = idx % NCOL, rest = idx / NCOL;
    const int gi = rest % GROUPS, m = rest / GROUPS;
    const int n = (blockIdx.x * GROUPS + gi) * NCOL + nl;
    if (m >= M || n >= N) continue;
    float v = GATED ? total(gi, 0, nl, m) : total(gi, nl / CP, nl % CP, m);
    if (scale_rows) v *= rstd[m];
    if (GATED) {
      float u = total(gi, 1, nl, m);
      if (scale_rows) u *= rstd[m];
      v = (v * (1.0f / (1.0f + expf(-v)))) * u;
    }
    if (bias && blockIdx.y == 0) v += bf16_to_f32(bias[n]);
    if (partial) Pp[(int64_t)m * N + n] = v;
    else Num<TC>::st(C + (int64_t)m * ldc + n, v);
  }
}

// The gated product of up to 16 rows, dealt EVENLY to the compute units.  A workgroup of the kernel above owns 16
// columns, whatever their number: the 8,960 columns of a 1.5B model make 560 workgroups for 256 compute units, and a
// unit that gets three of them streams half as much again as one that gets two.  Here the grid is a multiple of the
// number of compute units and workgroup b owns the columns [b N / G, (b + 1) N / G), up to NT tiles of 16 of the gate
// and as many of the up matrix: every unit streams the same bytes.  K is dealt to the 8 wavefronts and their parts are
// added exactly as above, so the results are the same bits.  How many columns a workgroup should own is a trade: every
// workgroup reads all rows of A (as much as M / 2 of its columns' weights), while more, smaller workgroups keep more
// loads on their way; the launcher's rule states what was measured.
// The same dealing serves a plain product of many columns (the head): TILES tiles of 16 columns of W a workgroup, the
// bias added to the sums.  GATED: the first half of the tiles is the gate's, the second the up matrix's.
template <int TILES, typename TC, bool GATED>
__global__ __launch_bounds__(SK_THREADS) void gemm_even_kernel(TC* __restrict__ C, int64_t ldc,
                                                               const bf16_t* __restrict__ A, int64_t lda,
                                                               const bf16_t* __restrict__ W,
                                                               const bf16_t* __restrict__ bias, int M, int N, int K,
                                                               int ksteps, NormIn norm_in) {
  static_assert(!GATED || TILES % 2 == 0, "as many tiles of the gate as of the up matrix");
  constexpr int PER = GATED ? TILES / 2 : TILES;             // tiles of one matrix
  __shared__ float red[SK_WAVES][TILES * 16][16 + 1];
  __shared__ float rstd[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int c0 = (int)(((int64_t)blockIdx.x * N) / gridDim.x), c1 = (int)(((int64_t)(blockIdx.x + 1) * N) / gridDim.x);
  const int cols = c1 - c0;                                  // <= PER * 16 by the launcher's choice of the grid
  const KRange<1> kr(wave, 0, ksteps, SK_WAVES, K);
  const bf16_t* wp[TILES];
  bool wok[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    const int cl = (t % PER) * 16 + r;                       // the lane's column within the workgroup's range
    wok[t] = cl < cols;
    wp[t] = W + ((int64_t)(wok[t] ? c0 + cl : 0) + (GATED && t >= PER ? (int64_t)N : 0)) * K + kr.shift;
  }
  const bf16_t* ap[1];
  bool aok[1];
  aok[0] = r < M;
  ap[0] = A + (int64_t)(aok[0] ? r : 0) * lda + kr.shift;
  f32x4 acc[TILES][1];
#pragma unroll
  for (int t = 0; t < TILES; ++t) acc[t][0] = f32x4{0.f, 0.f, 0.f, 0.f};
  NormInLoads in_loads;
  in_loads.load(norm_in, M, wave, lane);
  // steps of K asked for at once: fewer with more tiles, whose loads fill the registers
  skinny_accumulate<TILES, 1, (TILES <= 2 ? 4 : TILES <= 4 ? 2 : 1)>(acc, wp, wok, ap, aok, 0, kr.kend, kr.ke, g);
  in_loads.finish(norm_in, rstd, M, wave, lane);
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t * 16 + g * 4 + i][r] = acc[t][0][i];
  __syncthreads();
  const bool scale_rows = norm_in.sumsq != nullptr;
  for (int idx = threadIdx.x; idx < cols * M; idx += SK_THREADS) {
    const int cl = idx % cols, m = idx / cols;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < SK_WAVES; ++w) v += red[w][cl][m];            // in wavefront order, as in the kernel above
    if (scale_rows) v *= rstd[m];
    if (GATED) {
      float u = 0.f;
#pragma unroll
      for (int w = 0; w < SK_WAVES; ++w) u += red[w][PER * 16 + cl][m];
      if (scale_rows) u *= rstd[m];
      v = (v * (1.0f / (1.0f + expf(-v)))) * u;
    } else if (bias) {
      v += bf16_to_f32(bias[c0 + cl]);
    }
    Num<TC>::st(C + (int64_t)m * ldc + c0 + cl, v);
  }
}

// GaSkinnyNorm, what ga_gemm_skinny takes beside the product itself, is declared in ginfer_amd.h.

// Tiles of a product of M rows when the caller leaves the choice to the library: packed where they can be and
// full tiles would make fewer than 192 workgroups.  Measured on MI355X: a third faster where a product has few
// columns (1536: 96 workgroups of full tiles); no gain or a loss from 224 workgroups on (down projection of a 7B
// shape at 8 rows: 35 us with full tiles, 44 packed); the gated product was measured slower packed.
static int auto_pack(int M, int workgroups_of_full_tiles) {
  return (M <= 8 && workgroups_of_full_tiles < 192) ? 2 : 1;
}

// Columns that a workgroup of a product that folds the norm after it owns: the columns of a tile (16, or 8 when
// packed), or fewer where that spreads the product over more compute units.  Every such workgroup reads all rows of A,
// which with a long K is as much as its weights, and a compute unit takes in some 35 GB/s of such operands whatever it
// does with them: measured on MI355X (the 1.5B shape's down and output projections at 8 rows; 192 workgroups of 8 columns
// against 256 of 6): a decode step of 28 layers 1.745 -> 1.724 ms.  Never more workgroups than GA_FOLD_TARGET.
#define GA_FOLD_TARGET 256
// The gated product of up to 16 rows goes to the kernel that deals its columns evenly from this many (activation)
// columns on: a workgroup then has at least 8 of them.
#define GA_GATED_EVEN_MIN_COLUMNS 2048
// Its workgroups: the multiple of GA_FOLD_TARGET that comes nearest to 12 columns a workgroup with up to 4 rows (and up
// to 8 rows of a K of up to 2,048), 28 with up to 8 rows, 32 beyond, and never more than 48 (three tiles).  Measured on
// MI355X as replays of a graph that walks 28 layers' weights, in us, before -> after (columns a workgroup), at 1, 8 and
// 16 rows: 8,960 x 1,536: 16.7 -> 13.2 (12), 18.2 -> 15.7 (12), 20.5 -> 17.1 (35); 4,864 x 896: 8.5 -> 6.5 (10),
// 9.2 -> 7.2 (10), 10.0 -> 8.0 (19); 11,008 x 2,048: 22.7 -> 18.9 (11), 24.8 -> 23.3 (11), 27.2 -> 26.7 (43);
// 18,944 x 3,584: 57.4 -> 51.0 (13), 63.1 -> 60.3 (25), 71.7 -> 63.5 (37); 13,824 x 5,120: 63.9 -> 54.8 (11),
// 71.6 -> 63.6 (27), 82.3 -> 68.7 (27); 29,568 x 8,192: 183 -> 169 (12), 200 -> 191 (29), 234 -> 206 (29).
// The plain product of up to 16 rows and at least this many columns (the head) is dealt the same way, to workgroups of
// up to 6 tiles; 0: the kernel above keeps it.  Its thousands of small workgroups are even enough by their number, so
// less is gained: measured on MI355X at 151,936 x 1,536 with 32-bit sums out, in us, before -> after (columns a
// workgroup) at 1, 8 and 16 rows: 92.5 -> 86.0 (25), 109.9 -> 106.9 (75), 129.4 -> 113.5 (75); 152,064 x 3,584:
// 186 -> 183 (16), 237 -> 227 (85), 298 -> 240 (85); 152,064 x 8,192: 410 and 410 (16), 486 -> 481 (60), 625 -> 515 (85).
#define GA_PLAIN_EVEN_MIN_COLUMNS 16384
static int plain_even_workgroups(int M, int N, int K) {
  if (M <= 4 && K > 2048) return 0;
  const int target = M <= 4 ? 24 : 80;
  int rounds = (N + GA_FOLD_TARGET * target / 2) / (GA_FOLD_TARGET * target);
  if (rounds < 1) rounds = 1;
  while ((N + GA_FOLD_TARGET * rounds - 1) / (GA_FOLD_TARGET * rounds) > 96) ++rounds;
  return GA_FOLD_TARGET * rounds;
}
static int gated_even_workgroups(int M, int N, int K) {
  const int target = M <= 4 ? 12 : M <= 8 ? (K <= 2048 ? 12 : 28) : 32;
  int rounds = (N + GA_FOLD_TARGET * target / 2) / (GA_FOLD_TARGET * target);
  if (rounds < 1) rounds = 1;
  while ((N + GA_FOLD_TARGET * rounds - 1) / (GA_FOLD_TARGET * rounds) > 48) ++rounds;
  return GA_FOLD_TARGET * rounds;
}
static int fold_cols(int M, int N) {
  const int cp = 16 / auto_pack(M, (N + 15) / 16);
  const int full = (N + cp - 1) / cp;
  if (full >= GA_FOLD_TARGET) return cp;
  int cols = (N + GA_FOLD_TARGET - 1) / GA_FOLD_TARGET;          // as few columns as make GA_FOLD_TARGET workgroups
  return cols < 1 ? 1 : (cols > cp ? cp : cols);
}

// Partial sums a row gets from a product of M rows and N columns that feeds a norm.
extern "C" int ga_skinny_norm_parts(int M, int N) {
  const int cols = fold_cols(M, N);
  return (N + cols - 1) / cols;
}

// A [M, K] (row stride lda), W [N, K] contiguous, bias [N] or null.  grid_splits == 1: C [M, N] (row
// stride ldc) in bfloat16 or float.  grid_splits > 1: C is float [grid_splits][M][N], parts to be added
// by the consumer.  gated: W is [2N, K] (gate over up), C [M, N] = silu(A.gate^T) * (A.up^T), no bias, no
// grid split.  M <= 64, K a multiple of 8, rows 16-byte aligned.  nt in {1,2,4}, ks in {1,2,4,8}, pack in
// {1,2} (2: at most 8 rows); 0 lets the library choose.
extern "C" int ga_gemm_skinny(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias,
                              int M, int N, int K, int out_f32, int nt, int ks, int grid_splits, int gated, int pack,
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
    pack = auto_pack(M, (N + 15) / 16);          // what ga_skinny_norm_parts promised
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
  if (pack == 0) pack = (grid_splits == 1 && !gated) ? auto_pack(M, (N + groups * nt * 16 - 1) / (groups * nt * 16)) : 1;
  if (pack != 1 && (pack != 2 || M > 8)) return -2;
  const bool plain_even = !gated && grid_splits == 1 && !norm_out.residual && ks == SK_WAVES &&
                          N >= GA_PLAIN_EVEN_MIN_COLUMNS && plain_even_workgroups(M, N, K) > 0;
  if (mb == 1 && pack == 1 && ((gated && N >= GA_GATED_EVEN_MIN_COLUMNS) || plain_even)) {
    const int workgroups = gated ? gated_even_workgroups(M, N, K) : plain_even_workgroups(M, N, K);
    const int most = (N + workgroups - 1) / workgroups, per = (most + 15) / 16;      // tiles of one matrix
    const int ksteps = (K + 63) / 64;
    dim3 grid(workgroups), block(SK_THREADS);
#define LAUNCH_EVEN(TILES, TC, G)                                                                              \
  hipLaunchKernelGGL((gemm_even_kernel<TILES, TC, G>), grid, block, 0, stream, (TC*)C, ldc, (const bf16_t*)A, \
                     lda, (const bf16_t*)W, (const bf16_t*)bias, M, N, K, ksteps, norm_in)
#define PICK_EVEN(TC)                                                                                          \
  if (gated) {                                                                                                 \
    if (per == 1) LAUNCH_EVEN(2, TC, true); else if (per == 2) LAUNCH_EVEN(4, TC, true); else LAUNCH_EVEN(6, TC, true); \
  } else {                                                                                                     \
    if (per <= 2) LAUNCH_EVEN(2, TC, false); else if (per <= 4) LAUNCH_EVEN(4, TC, false); else LAUNCH_EVEN(6, TC, false); \
  }
    if (out_f32) { PICK_EVEN(float) } else { PICK_EVEN(bf16_t) }
#undef PICK_EVEN
#undef LAUNCH_EVEN
    return GA_CHECK_LAUNCH();
  }
  const int cp = 16 / pack;
  const int ncol = gated ? cp : nt * cp;
  const int ksteps = (K + 63) / 64;
  dim3 grid((N + groups * ncol - 1) / (groups * ncol), grid_splits), block(SK_THREADS);
  int fcols = 0;
  if (norm_out.residual) {
    fcols = fold_cols(M, N);
    grid.x = (N + fcols - 1) / fcols;
  }
#define LAUNCH(NT, MB, KS, TC, G, PK)                                                                     \
  hipLaunchKernelGGL((gemm_skinny_kernel<NT, MB, KS, TC, G, PK>), grid, block, 0, stream, (TC*)C, ldc,   \
                     (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, M, N, K, ksteps,      \
                     norm_in, norm_out, fcols)
#define PICK_KS(NT, MB, TC, G, PK)                                                                        \
  switch (ks) {                                                                                           \
    case 1: LAUNCH(NT, MB, 1, TC, G, PK); break;                                                          \
    case 2: LAUNCH(NT, MB, 2, TC, G, PK); break;                                                          \
    case 4: LAUNCH(NT, MB, 4, TC, G, PK); break;                                                          \
    default: LAUNCH(NT, MB, 8, TC, G, PK); break;                                                         \
  }
#define PICK_MB(NT, TC, G)                                                                                \
  switch (mb) {                                                                                           \
    case 1:                                                                                               \
      if (pack == 2) { PICK_KS(NT, 1, TC, G, 2) } else { PICK_KS(NT, 1, TC, G, 1) }                       \
      break;                                                                                              \
    case 2: PICK_KS(NT, 2, TC, G, 1) break;                                                               \
    case 3: PICK_KS(NT, 3, TC, G, 1) break;                                                               \
    default: PICK_KS(NT, 4, TC, G, 1) break;                                                              \
  }
#define PICK_NT(TC)                                                                                       \
  switch (nt) {                                                                                           \
    case 1: PICK_MB(1, TC, false) break;                                                                  \
    case 2: PICK_MB(2, TC, false) break;                                                                  \
    default: PICK_MB(4, TC, false) break;                                                                 \
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
// ginfer/core/op/kernels/cuda/store_kvcache_kernel.cu:19-30).  A wavefront group owns a UNIT of 2 CP output
// columns as two tiles of CP (16, or 8 when packed): for a q or k head the columns j0..j0+CP-1 and their
// rotation partners j0+half..; for a v head 2 CP consecutive columns.  head_dim a multiple of 32,
// rotary_dim == head_dim.  HALF (with more than 16 rows of A, where tiles cannot be packed): a tile holds 8 rows
// of W and nothing in its other half, so that twice the workgroups share the product; this product has too few
// columns to fill the chip otherwise, and its K cannot be split over workgroups (the epilogue needs whole sums).
template <int MB, int KS, int PACK, bool HALF>
__global__ __launch_bounds__(SK_THREADS) void qkv_rope_skinny_kernel(
    bf16_t* __restrict__ q_out, const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W,
    const bf16_t* __restrict__ bias, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int64_t* __restrict__ slot_mapping, bf16_t* __restrict__ k_pages,
    bf16_t* __restrict__ v_pages, int M, int K, int nh, int nkv, int hd, int page_size, int write_kv,
    int ksteps, NormIn norm_in, int ucols) {
  static_assert(PACK == 1 || MB == 1, "a packed tile holds at most 8 rows of A");
  static_assert(PACK == 1 || !HALF, "a tile is packed or half empty, not both");
  __shared__ float red[SK_WAVES][32][MB * 16 + 1];
  __shared__ float rstd[16];
  using P = Packed<PACK>;
  constexpr int CP = HALF ? 8 : P::CP;
  constexpr int GROUPS = SK_WAVES / KS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int grp = wave / KS, ks = wave % KS;
  // a unit's two tiles hold `ucols` (<= CP) columns each: fewer than a tile's where that spreads the product over more
  // compute units (the lanes of the other columns load nothing)
  const int half = hd >> 1, upq = half / ucols;         // units per q or k head
  const int upv = hd / (2 * ucols);                     // units per v head
  const int qk_units = (nh + nkv) * upq, units = qk_units + nkv * upv;
  const int unit = blockIdx.x * GROUPS + grp;
  const bool unit_ok = unit < units;
  // first rows of the unit's two tiles
  int row0 = 0, row1 = 0;
  if (unit_ok) {
    if (unit < qk_units) {
      row0 = (unit / upq) * hd + (unit % upq) * ucols;
      row1 = row0 + half;
    } else {
      const int u = unit - qk_units;
      row0 = (nh + nkv) * hd + u * 2 * ucols;
      row1 = row0 + ucols;
    }
  }
  const KRange<PACK> kr(ks * PACK, P::seg(r), ksteps, KS * PACK, K);
  const int shift = kr.shift;
  const int wrow = HALF ? (r & 7) : P::col(r);
  const bool lane_ok = unit_ok && (!HALF || r < 8) && wrow < ucols;
  const bf16_t* wp[2] = {W + (int64_t)(row0 + wrow) * K + shift, W + (int64_t)(row1 + wrow) * K + shift};
  const bool wok[2] = {lane_ok, lane_ok};
  const bf16_t* ap[MB];
  bool aok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + P::col(r);
    aok[mb] = m < M;
    ap[mb] = A + (int64_t)(aok[mb] ? m : 0) * lda + shift;
  }
  // What the epilogue needs from memory (position, slot, cosine and sine, bias) is asked for now, so that
  // it arrives while the weights stream: an epilogue item is (unit of the workgroup, column, row of A).
  constexpr int MROWS = PACK == 1 ? MB * 16 : CP;
  constexpr int ITEMS = (GROUPS * CP * MROWS + SK_THREADS - 1) / SK_THREADS;
  int64_t e_slot[ITEMS];
  float e_cos[ITEMS], e_sin[ITEMS], e_blo[ITEMS], e_bhi[ITEMS];
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int idx = threadIdx.x + it * SK_THREADS;
    const int nl = idx % ucols, rest = idx / ucols;
    const int gi = rest % GROUPS, m = rest / GROUPS;
    const int u = blockIdx.x * GROUPS + gi;
    e_slot[it] = -1;
    e_cos[it] = 1.f;
    e_sin[it] = e_blo[it] = e_bhi[it] = 0.f;
    if (m < M && u < units) {
      if (write_kv) e_slot[it] = slot_mapping[m];
      if (u < qk_units) {
        const int head = u / upq, j = (u % upq) * ucols + nl;
        const int p = positions[m];
        e_cos[it] = cos_t[(int64_t)p * half + j];
        e_sin[it] = sin_t[(int64_t)p * half + j];
        if (bias) {
          e_blo[it] = bf16_to_f32(bias[head * hd + j]);
          e_bhi[it] = bf16_to_f32(bias[head * hd + j + half]);
        }
      } else if (bias) {
        const int v = u - qk_units;
        const int at = (nh + nkv + v / upv) * hd + (v % upv) * 2 * ucols + nl;
        e_blo[it] = bf16_to_f32(bias[at]);
        e_bhi[it] = bf16_to_f32(bias[at + ucols]);
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
  skinny_accumulate<2, MB>(acc, wp, wok, ap, aok, 0, kr.kend, kr.ke, g);
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
    const int nl = idx % ucols, rest = idx / ucols;
    const int gi = rest % GROUPS, m = rest / GROUPS;
    const int u = blockIdx.x * GROUPS + gi;
    if (m >= M || u >= units) continue;
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int w = 0; w < KS; ++w)
#pragma unroll
      for (int q = 0; q < PACK; ++q) {
        const int col = PACK == 1 ? m : q * CP + m;
        lo += red[gi * KS + w][q * CP + nl][col];
        hi += red[gi * KS + w][16 + q * CP + nl][col];
      }
    if (scale_rows) {
      lo *= rstd[m];
      hi *= rstd[m];
    }
    lo += e_blo[it];
    hi += e_bhi[it];
    const int64_t slot = e_slot[it];
    int64_t page = 0, off = 0;
    if (slot >= 0) slot_page(slot, page_size, page, off);
    if (u < qk_units) {
      const int head = u / upq, j = (u % upq) * ucols + nl;
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
      const int gh = v / upv, d = (v % upv) * 2 * ucols + nl;
      bf16_t* o = v_pages + ((page * nkv + gh) * (int64_t)hd + d) * page_size + off;
      o[0] = f32_to_bf16(lo);
      o[(int64_t)ucols * page_size] = f32_to_bf16(hi);
    }
  }
}

// q_out [M, nh*hd]; A [M, K] (row stride lda); W [(nh + 2 nkv) hd, K]; bias [(nh + 2 nkv) hd] or null;
// positions int32 [M]; cos_t, sin_t float [positions, hd/2]; slot_mapping int64 [M] (-1: no cache write);
// k_pages [pages, nkv, page_size, hd], v_pages [pages, nkv, hd, page_size].  norm: null, or the sums of the
// norm whose (h * g) the rows of A are (its in_ fields only).  pack: 0 (the library chooses), 1 or 2.
#define GA_QKV_SPREAD_BELOW 192
extern "C" int ga_qkv_rope_skinny(void* q_out, const void* A, int64_t lda, const void* W, const void* bias,
                                  const void* positions, const void* cos_t, const void* sin_t,
                                  const void* slot_mapping, void* k_pages, void* v_pages, int M, int K, int nh,
                                  int nkv, int hd, int page_size, int write_kv, int pack, const GaSkinnyNorm* norm,
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
  if (pack == 0) pack = auto_pack(M, (nh + 2 * nkv) * hd / 32);
  if (pack != 1 && (pack != 2 || M > 8)) return -2;
  const int ks = 8, groups = SK_WAVES / ks;
  // with more than 8 rows and so few columns that full tiles leave most of the chip idle: half tiles (measured on
  // MI355X: 64 rows 11.4 us against 15.9 with 64 workgroups of full tiles; with 144 of them, slower)
  const bool half_tiles = pack == 1 && M > 8 && (nh + 2 * nkv) * hd / 32 < 128;
  // columns of a unit's tile: all of a tile's, or half of them where a packed tile's 8 would leave the product on fewer
  // than GA_QKV_SPREAD_BELOW workgroups (2,048 columns of a K of 1,536 at 8 rows: 128 workgroups of 8 + 8 columns
  // 7.15 us in a decode step, 256 of 4 + 4 see the measurement beside the macro)
  int ucols = half_tiles ? 8 : 16 / pack;
  if (pack == 2 && (nh + 2 * nkv) * hd / (2 * ucols) < GA_QKV_SPREAD_BELOW && (hd / 2) % (ucols / 2) == 0) ucols /= 2;
  const int units = (nh + 2 * nkv) * hd / (2 * ucols);
  const int ksteps = (K + 63) / 64;
  dim3 grid((units + groups - 1) / groups), block(SK_THREADS);
#define LAUNCH(MB, PK, HF)                                                                                \
  hipLaunchKernelGGL((qkv_rope_skinny_kernel<MB, 8, PK, HF>), grid, block, 0, stream, (bf16_t*)q_out,    \
                     (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, (const int32_t*)positions, \
                     (const float*)cos_t, (const float*)sin_t, (const int64_t*)slot_mapping, (bf16_t*)k_pages, \
                     (bf16_t*)v_pages, M, K, nh, nkv, hd, page_size, write_kv, ksteps, norm_in, ucols)
  switch (mb) {
    case 1:
      if (pack == 2) LAUNCH(1, 2, false); else if (half_tiles) LAUNCH(1, 1, true); else LAUNCH(1, 1, false);
      break;
    case 2:
      if (half_tiles) LAUNCH(2, 1, true); else LAUNCH(2, 1, false);
      break;
    case 3:
      if (half_tiles) LAUNCH(3, 1, true); else LAUNCH(3, 1, false);
      break;
    default:
      if (half_tiles) LAUNCH(4, 1, true); else LAUNCH(4, 1, false);
      break;
  }
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
