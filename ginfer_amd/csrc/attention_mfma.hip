// Paged attention on the matrix cores (bfloat16 storage; 32-bit scores, softmax and accumulators),
// compiled for one head size: -DHEAD_DIM=<multiple of 16, at most 256>.
//
// Both kernels here share one inner loop.  A wavefront owns up to 16*NB "columns"; a column is one
// (token, query head) pair, all columns of a wavefront reading the same kv head of the same request.
//   decode kernel : columns = the query heads of one kv-head group for ONE token; the keys are split
//                   over blockIdx.z, partial (max, sum, output) go to a workspace and a second kernel
//                   combines the splits in ascending order.  Replaces the reference's unsplit,
//                   one-head-per-block kernel (ginfer/core/op/kernels/cuda/page_attn_kernel/
//                   flash_gqa_varlen_decode_kvcache.cu:272-335), in which every head of a group re-reads
//                   the same keys.
//   prefill kernel: columns = 16*NB consecutive tokens of one request's portion, one head per
//                   wavefront, the heads of a kv-head group side by side in a workgroup so that they
//                   stream the same keys together (flash_gqa_varlen_kernel.cu:420-512 is the reference's).
// Mask: column with position p sees keys c in [max(0, p - window + 1), p]  (flash_gqa_varlen_kernel.cu:
// 202-222 in absolute positions).  score = (q . k) * scale on the 32-bit product; online softmax over
// tiles of 32 keys at absolute multiples of 32.
//
// Matrix-core mapping (v_mfma_f32_16x16x32_bf16: D[m][n] += sum_k A[m][k] B[n][k]; lane l supplies row
// l%16 and k-slots (l/16)*8..+7 of both operands and receives D[(l/16)*4+i][l%16], i = 0..3):
//   S^T = K Q^T : A = 16 keys x 32 dims of K (one 16-byte load per lane straight from the page),
//                 B = 16 columns x 32 dims of Q (kept in registers); two such products per tile.
//                 Row m of product t holds key 8*(m/4) + 4*t + m%4 of the tile, so a lane ends up with
//                 the scores of the 8 CONSECUTIVE keys 8*(l/16)..+7 of its column,
//   O^T += V^T P: which is exactly the k-slot layout of operand B for P, with no shuffle; operand A is
//                 16 dims x 8 consecutive keys of V^T: one 16-byte load per lane because the cache keeps
//                 values transposed inside a page ([page][kv_head][dim][slot]).
// The decode kernel and the first prefill kernel stage nothing through LDS: each operand element is loaded
// once per wavefront, and the heads of a group that run side by side hit the same lines in the vector cache.
// The second prefill kernel (head sizes 64, 128, 256) has one wavefront load each tile into LDS for all heads.
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size: multiples of 16 up to 256");

constexpr int HD = HEAD_DIM;
constexpr int KB = (HD + 31) / 32;   // 32-dim blocks of the q.k product (the last may be half empty)
constexpr int DB = HD / 16;          // 16-dim blocks of the output
constexpr int PREFILL_NB = HD <= 128 ? 2 : 1;
// Measured on MI355X (12 heads in 2 groups, head size 128, prompts of 2k to 16k tokens): workgroups of 8
// wavefronts with one set of key and value registers in flight are fastest (66 us at 2k, 530 us at 8k).  4
// wavefronts (one per SIMD, 512 registers each) take 78 and 638 us, with one set or two: the loads' latency is
// not what the kernel waits for; its vector instructions (softmax) take 1.7 times the issue time of its matrix
// products, and two wavefronts per SIMD overlap the two.
#ifndef PREFILL_DEPTH
#define PREFILL_DEPTH 1              // sets of key and value registers in flight in the prefill kernel
#endif
#ifndef DECODE_DEPTH
#define DECODE_DEPTH 1               // ... and in the decode kernel (2 was measured no faster from 1k to 128k tokens)
#endif
#ifndef PREFILL_WAVES
#define PREFILL_WAVES 8              // wavefronts of a prefill workgroup
#endif

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

// The kernels keep scores, running maxima and the maxima of partial results in units of log2(e): the
// launchers multiply the score scale by LOG2E once, and every exponential is a bare exp2.
#define LOG2E 1.4426950408889634f
#define LAZY_MAX 8.0f

// the bare v_exp_f32: arguments here are differences to a running maximum (<= 0, or -inf), for which the
// library routine's extra steps for denormal results buy nothing
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ bf16x8 zero8() {
  uint4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}
__device__ __forceinline__ bf16x8 load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

// The pages of a tile of 32 keys, the same for every lane: up to four consecutive entries of the block table
// (a page holds at least 8 keys), read with scalar loads, which wait on a counter of their own: a vector load
// of a page id would have to be waited for together with every key and value load issued before it.
struct TilePages {
  int p0, p1, p2, p3;
};
__device__ __forceinline__ int table_entry(const int32_t* __restrict__ bt, int table_width, int idx) {
  return bt[idx < table_width ? idx : table_width - 1];   // entries past the tile's last page are never picked
}
__device__ __forceinline__ void lookup_pages(TilePages& tp, const int32_t* __restrict__ bt, int table_width,
                                             int ps_shift, int k0) {
  const int first = k0 >> ps_shift;
  tp.p0 = table_entry(bt, table_width, first);
  tp.p1 = table_entry(bt, table_width, first + 1);
  tp.p2 = table_entry(bt, table_width, first + 2);
  tp.p3 = table_entry(bt, table_width, first + 3);
}

// What a lane reads of every tile: its two K rows (products t = 0, 1) and its 8-key piece of V^T, as offsets in the
// tile and as the one of the tile's pages that holds them.
struct PageChoice {
  bool is1, is2, is3;
};
struct LaneKeys {
  int koff[2], voff;
  PageChoice ksel[2], vsel;
};
__device__ __forceinline__ PageChoice page_choice(int offset, int ps_shift) {
  const int sel = offset >> ps_shift;
  return PageChoice{sel == 1, sel == 2, sel == 3};
}
__device__ __forceinline__ LaneKeys lane_keys(int ps_shift, int c, int g) {
  LaneKeys lk;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    lk.koff[t] = 8 * (c >> 2) + 4 * t + (c & 3);
    lk.ksel[t] = page_choice(lk.koff[t], ps_shift);
  }
  lk.voff = 8 * g;
  lk.vsel = page_choice(lk.voff, ps_shift);
  return lk;
}
__device__ __forceinline__ int pick_page(const TilePages& tp, const PageChoice& ch) {
  // the page ids pass through empty statements that pin them as values in scalar registers: a select between
  // loads of the four would be turned into one load at a selected address, of an array in scratch memory
  int p0 = tp.p0, p1 = tp.p1, p2 = tp.p2, p3 = tp.p3;
  asm("" : "+s"(p0));
  asm("" : "+s"(p1));
  asm("" : "+s"(p2));
  asm("" : "+s"(p3));
  int p = p0;
  p = ch.is1 ? p1 : p;
  p = ch.is2 ? p2 : p;
  p = ch.is3 ? p3 : p;
  return p;
}

// K operands of one tile of 32 keys: [product t][32-dim block].  In an edge tile (one that reaches past kv_min or
// kv_max) the keys outside the range take page 0, which is always there: their pages may be gone (-1) or lie past
// the table; what is read for them is masked (scores) or cleared (values).  Rows of the cache are counted in 32
// bits (the caller checks that pages * nkv * page_size fits).
__device__ __forceinline__ void load_k_tile(bf16x8 (&kr)[2][KB], const bf16_t* __restrict__ k_pages,
                                            const TilePages& tp, const LaneKeys& lk, int kvh, int nkv, int ps_shift,
                                            int k0, bool edge, int kv_min, int kv_max, int g) {
  const int ps = 1 << ps_shift;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int key = k0 + lk.koff[t];
    int page = pick_page(tp, lk.ksel[t]);
    if (edge) page = (key >= kv_min && key <= kv_max) ? page : 0;
    const int row = ((page * nkv + kvh) << ps_shift) + (key & (ps - 1));
    const bf16_t* kp = k_pages + (int64_t)row * HD + g * 8;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      if (HD % 32 == 0 || kb * 32 + g * 8 < HD) kr[t][kb] = load8(kp + kb * 32);
      else kr[t][kb] = zero8();
    }
  }
}

// V^T operands of one tile: [16-dim block]; the lane loads dims db*16 + c, keys k0 + 8g .. + 7 (one page: a page
// holds a multiple of 8 keys).  A piece that straddles an end of the range has a live key and so a live page.
__device__ __forceinline__ void load_v_tile(bf16x8 (&vr)[DB], const bf16_t* __restrict__ v_pages,
                                            const TilePages& tp, const LaneKeys& lk, int kvh, int nkv, int ps_shift,
                                            int k0, bool edge, int kv_min, int kv_max, int c) {
  const int ps = 1 << ps_shift;
  const int kbase = k0 + lk.voff;
  int page = pick_page(tp, lk.vsel);
  if (edge) page = (kbase + 7 >= kv_min && kbase <= kv_max) ? page : 0;
  const int row = (page * nkv + kvh) * HD + c;
  const bf16_t* vp = v_pages + ((int64_t)row << ps_shift) + (kbase & (ps - 1));
#pragma unroll
  for (int db = 0; db < DB; ++db) vr[db] = load8(vp + (int64_t)db * 16 * ps);
}

// The steps of one tile of 32 keys starting at k0, shared by the loops that keep the tile's operands in registers
// and the one that reads them from LDS.
// ---- scores: S^T = K Q^T
template <int NB>
__device__ __forceinline__ void tile_scores(f32x4 (&s)[NB][2], const bf16x8 (&kr)[2][KB], const bf16x8 (&q)[NB][KB]) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    s[nb][0] = f32x4{0.f, 0.f, 0.f, 0.f};
    s[nb][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        s[nb][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kr[t][kb], q[nb][kb], s[nb][t], 0, 0, 0);
}

// ---- mask and online softmax; the lane holds keys k0 + 8g + j, j = 0..7, of column c.  The running max is
// kept in scaled units; the scale rides on the exponent's multiply-add.  An empty column (no query: its q is
// zero) goes along unmasked in interior tiles; nothing of it is ever written.
template <int NB>
__device__ __forceinline__ void tile_softmax(bf16x8 (&pb)[NB], f32x4 (&s)[NB][2], f32x4 (&o)[NB][DB],
                                             float (&m)[NB], float (&l)[NB], const int (&cpos)[NB],
                                             const int (&clo)[NB], int full_lo, int full_hi, int k0, float scale,
                                             int g) {
  const bool interior = k0 >= full_lo && k0 + 31 <= full_hi;      // the same for the whole wavefront
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    if (!interior) {
      // The lane's key j is live where lo <= j <= hi: two subtractions here, none on the path without a mask.  The
      // scores are masked where they lie (a select: what was read for a dead key is dropped), so that the path
      // without a mask copies nothing.
      const int lo = clo[nb] - (k0 + 8 * g), hi = cpos[nb] - (k0 + 8 * g);
#pragma unroll
      for (int j = 0; j < 8; ++j) s[nb][j >> 2][j & 3] = (j >= lo && j <= hi) ? s[nb][j >> 2][j & 3] : -INFINITY;
    }
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      sv[j] = s[nb][j >> 2][j & 3];
      mx = fmaxf(mx, sv[j]);
    }
    // The running max is raised lazily: only when some score of the tile exceeds it by more than
    // LAZY_MAX (in log2 units), which after the first tiles is rare.  Until then exponentials may reach
    // 2^LAZY_MAX, harmless in 32-bit sums, and the tile costs no exchange between lanes: the four lanes
    // of a column keep partial sums of their own keys (added up once, by finish_sums, after the loop).
    if (__any(mx * scale > m[nb] + LAZY_MAX)) {
      mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
      const float m_new = fmaxf(m[nb], mx * scale);
      if (m_new != -INFINITY) {
        const float alpha = fast_exp2(m[nb] - m_new);      // exp2(-inf) = 0 the first time
        l[nb] *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db) o[nb][db] *= alpha;
      }
      m[nb] = m_new;
    }
    // A column that has seen no key yet has m == -inf and only dead keys (-inf) in this tile: with 0 in
    // place of m every exponent is -inf and every p is 0, without a branch.
    const float m_use = m[nb] == -INFINITY ? 0.f : m[nb];
    float sum = 0.f;
    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p[j] = fast_exp2(__builtin_fmaf(sv[j], scale, -m_use));
      sum += p[j];
    }
    l[nb] += sum;
    // two values to a conversion (v_cvt_pk_bf16_f32), round to nearest even
    union { bf16x8 v; bf16x2 h[4]; } packed;
#pragma unroll
    for (int j = 0; j < 4; ++j) packed.h[j] = __builtin_convertvector(f32x2{p[2 * j], p[2 * j + 1]}, bf16x2);
    pb[nb] = packed.v;
  }
}

// ---- output: O^T += V^T P.  In a tile that reaches past the ends of the key range the values read for dead
// keys (anything: the slot may never have been written) are cleared first: 0 * NaN is not 0.
template <int NB>
__device__ __forceinline__ void tile_output(f32x4 (&o)[NB][DB], bf16x8 (&vr)[DB], const bf16x8 (&pb)[NB], int kv_min,
                                            int kv_max, int k0, int g) {
  if (k0 < kv_min || k0 + 31 > kv_max) {
    const int kbase = k0 + 8 * g;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      union { bf16x8 v; bf16_t e[8]; } u;
      u.v = vr[db];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (kbase + j < kv_min || kbase + j > kv_max) u.e[j] = 0;
      vr[db] = u.v;
    }
  }
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      o[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vr[db], pb[nb], o[nb][db], 0, 0, 0);
}

// One tile with its operands in the registers kr and vr.  As soon as the products that read kr (then vr) have
// been issued the registers are refilled with the tile k_refill (< 0: none), whose pages pg holds; after that pg
// takes the pages of the tile k_lookup (< 0: none).
template <int NB>
__device__ __forceinline__ void attend_one_tile(f32x4 (&o)[NB][DB], float (&m)[NB], float (&l)[NB],
                                                const bf16x8 (&q)[NB][KB], const int (&cpos)[NB],
                                                const int (&clo)[NB], bf16x8 (&kr)[2][KB], bf16x8 (&vr)[DB],
                                                TilePages& pg, const LaneKeys& lk,
                                                const bf16_t* __restrict__ k_pages,
                                                const bf16_t* __restrict__ v_pages,
                                                const int32_t* __restrict__ bt, int table_width, int kvh, int nkv,
                                                int ps_shift, int kv_min, int kv_max, int full_lo, int full_hi,
                                                int k0, int k_refill, int k_lookup, float scale, int c, int g) {
  f32x4 s[NB][2];
  tile_scores<NB>(s, kr, q);
  const bool refill_edge = k_refill < kv_min || k_refill + 31 > kv_max;
  if (k_refill >= 0) load_k_tile(kr, k_pages, pg, lk, kvh, nkv, ps_shift, k_refill, refill_edge, kv_min, kv_max, g);
  bf16x8 pb[NB];
  tile_softmax<NB>(pb, s, o, m, l, cpos, clo, full_lo, full_hi, k0, scale, g);
  tile_output<NB>(o, vr, pb, kv_min, kv_max, k0, g);
  if (k_refill >= 0) load_v_tile(vr, v_pages, pg, lk, kvh, nkv, ps_shift, k_refill, refill_edge, kv_min, kv_max, c);
  if (k_lookup >= 0) lookup_pages(pg, bt, table_width, ps_shift, k_lookup);
}

// Attends columns to the key tiles tile_begin, tile_begin + tile_stride, ... < tile_end (multiples of 32).
// kv_min..kv_max is the inclusive range of keys that any column of the wavefront may see; full_lo..full_hi
// the range that EVERY live column sees (tiles inside it need no mask).  The loop is software-pipelined
// DEPTH tiles deep: DEPTH sets of operand registers are filled ahead, each refilled with the tile DEPTH
// further on as soon as the products that read it have been issued, and the pages of a tile are looked up
// DEPTH tiles before its loads; so no load waits for a look-up and each has (nearly) DEPTH tiles' products and
// softmax to arrive in.  DEPTH 2 costs a second set of registers.
template <int NB, int DEPTH>
__device__ __forceinline__ void attend_tiles(f32x4 (&o)[NB][DB], float (&m)[NB], float (&l)[NB],
                                             const bf16x8 (&q)[NB][KB], const int (&cpos)[NB],
                                             const int (&clo)[NB], const bf16_t* __restrict__ k_pages,
                                             const bf16_t* __restrict__ v_pages,
                                             const int32_t* __restrict__ bt, int table_width, int kvh, int nkv,
                                             int ps_shift, int kv_min, int kv_max, int full_lo, int full_hi,
                                             int tile_begin, int tile_end, int tile_stride, float scale) {
  static_assert(DEPTH == 1 || DEPTH == 2, "one or two sets of operand registers");
  const int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  // the same in every lane of the wavefront, by the callers' construction: said so, the loop and its branches
  // run on the scalar unit and the page ids come through scalar loads
  tile_begin = __builtin_amdgcn_readfirstlane(tile_begin);
  tile_end = __builtin_amdgcn_readfirstlane(tile_end);
  tile_stride = __builtin_amdgcn_readfirstlane(tile_stride);
  kv_min = __builtin_amdgcn_readfirstlane(kv_min);
  kv_max = __builtin_amdgcn_readfirstlane(kv_max);
  full_lo = __builtin_amdgcn_readfirstlane(full_lo);
  full_hi = __builtin_amdgcn_readfirstlane(full_hi);
  if (tile_begin >= tile_end) return;
  const LaneKeys lk = lane_keys(ps_shift, c, g);
  TilePages pg[DEPTH];
  bf16x8 kr[DEPTH][2][KB], vr[DEPTH][DB];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const int k0 = tile_begin + d * tile_stride;
    if (k0 < tile_end) {
      const bool edge = k0 < kv_min || k0 + 31 > kv_max;
      lookup_pages(pg[d], bt, table_width, ps_shift, k0);
      load_k_tile(kr[d], k_pages, pg[d], lk, kvh, nkv, ps_shift, k0, edge, kv_min, kv_max, g);
      load_v_tile(vr[d], v_pages, pg[d], lk, kvh, nkv, ps_shift, k0, edge, kv_min, kv_max, c);
    }
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const int k0 = tile_begin + (DEPTH + d) * tile_stride;
    if (k0 < tile_end) lookup_pages(pg[d], bt, table_width, ps_shift, k0);
  }
  for (int kbase = tile_begin; kbase < tile_end; kbase += DEPTH * tile_stride) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int k0 = kbase + d * tile_stride;
      if (k0 < tile_end) {
        const int k_refill = k0 + DEPTH * tile_stride, k_lookup = k0 + 2 * DEPTH * tile_stride;
        attend_one_tile<NB>(o, m, l, q, cpos, clo, kr[d], vr[d], pg[d], lk, k_pages, v_pages, bt, table_width, kvh,
                            nkv, ps_shift, kv_min, kv_max, full_lo, full_hi, k0, k_refill < tile_end ? k_refill : -1,
                            k_lookup < tile_end ? k_lookup : -1, scale, c, g);
      }
    }
  }
}

// after attend_tiles: the four lanes of a column add up their partial sums
template <int NB>
__device__ __forceinline__ void finish_sums(float (&l)[NB]) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    l[nb] += __shfl_xor(l[nb], 16, WAVE);
    l[nb] += __shfl_xor(l[nb], 32, WAVE);
  }
}

template <int NB>
__device__ __forceinline__ void init_state(f32x4 (&o)[NB][DB], float (&m)[NB], float (&l)[NB]) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    m[nb] = -INFINITY;
    l[nb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) o[nb][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
}

// q operand of one column: 32-dim blocks of the column's query row, this lane's 8 dims
__device__ __forceinline__ void load_q(bf16x8 (&q)[KB], const bf16_t* row /* null: empty column */, int g) {
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    q[kb] = zero8();
    if (row && kb * 32 + g * 8 < HD) q[kb] = load8(row + kb * 32 + g * 8);
  }
}

// ----------------------------------------------------------------------------- decode
// grid (decode tokens, nkv * head_blocks, splits); a workgroup of DEC_WAVES wavefronts shares one split:
// wavefront w takes the key tiles w, w + DEC_WAVES, ... of the split, and the states meet in LDS.
// part_o: [n_tokens][nh][splits][HD] float; part_ml: [n_tokens][nh][splits][2] float (max, sum).
// With one split the normalised result goes straight to `out`.
#define DEC_WAVES 4

__global__ __launch_bounds__(64 * DEC_WAVES) void attn_decode_split_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, float* __restrict__ part_o, float* __restrict__ part_ml,
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, const int32_t* __restrict__ block_table, int table_width,
    const int4* __restrict__ decode_info, int nh, int nkv, int head_blocks, int ps_shift, int window,
    float scale, int split_keys, int num_splits) {
  __shared__ float o_s[DEC_WAVES][HD][17];
  __shared__ float m_s[DEC_WAVES][16], l_s[DEC_WAVES][16], mx_s[16], lsum_s[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  const int ti = blockIdx.x, split = blockIdx.z;
  const int kvh = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int group = nh / nkv;
  const int4 info = decode_info[ti];       // (row of the step, position, entry of the block table, -): one load
  const int t = info.x, pos = info.y;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const bool col_ok = hb * 16 + c < group;
  const int head = kvh * group + hb * 16 + c;

  f32x4 o[1][DB];
  float m[1], l[1];
  init_state<1>(o, m, l);
  const int begin = (lo / 32) * 32 + split * split_keys;
  if (begin <= pos) {
    int end = begin + split_keys;
    if (end > pos + 1) end = ((pos + 32) / 32) * 32;
    bf16x8 qr[1][KB];
    load_q(qr[0], col_ok ? q + (int64_t)t * q_stride + (int64_t)head * HD : nullptr, g);
    const int cpos[1] = {col_ok ? pos : -1}, clo[1] = {lo};
    const int32_t* bt = block_table + (int64_t)__builtin_amdgcn_readfirstlane(info.z) * table_width;
    // every live column of a decode wavefront sees the same keys: lo..pos
    attend_tiles<1, DECODE_DEPTH>(o, m, l, qr, cpos, clo, k_pages, v_pages, bt, table_width, kvh, nkv, ps_shift, lo,
                                  pos, lo, pos, begin + 32 * wave, end, 32 * DEC_WAVES, scale);
    finish_sums<1>(l);
  }
  // the wavefronts' states meet: common max, rescaled sums and outputs added in wavefront order
  if (g == 0) {
    m_s[wave][c] = m[0];
    l_s[wave][c] = l[0];
  }
  __syncthreads();
  float mx = -INFINITY;
#pragma unroll
  for (int w = 0; w < DEC_WAVES; ++w) mx = fmaxf(mx, m_s[w][c]);
  const float f = (m[0] == -INFINITY) ? 0.f : fast_exp2(m[0] - mx);
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i) o_s[wave][db * 16 + g * 4 + i][c] = o[0][db][i] * f;
  __syncthreads();
  // per column: the common max and the sum of the rescaled sums, once (the outputs in o_s are rescaled already)
  if (threadIdx.x < 16) {
    const int cc = threadIdx.x;
    float mcc = -INFINITY;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) mcc = fmaxf(mcc, m_s[w][cc]);
    float lsum = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) {
      const float mw = m_s[w][cc];
      if (mw != -INFINITY) lsum += l_s[w][cc] * fast_exp2(mw - mcc);
    }
    mx_s[cc] = mcc;
    lsum_s[cc] = lsum;
  }
  __syncthreads();
  const int64_t slot_base = ((int64_t)ti * nh + kvh * group + hb * 16) * num_splits + split;
  for (int idx = threadIdx.x; idx < 16 * HD; idx += 64 * DEC_WAVES) {
    const int cc = idx / HD, d = idx % HD;
    if (hb * 16 + cc >= group) continue;
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) acc += o_s[w][d][cc];
    if (num_splits == 1) {
      out[(int64_t)t * out_stride + (int64_t)(kvh * group + hb * 16 + cc) * HD + d] = f32_to_bf16(acc * (1.f / lsum_s[cc]));
    } else {
      const int64_t slot = slot_base + (int64_t)cc * num_splits;
      part_o[slot * HD + d] = acc;
      if (d == 0) {
        part_ml[slot * 2] = mx_s[cc];
        part_ml[slot * 2 + 1] = lsum_s[cc];
      }
    }
  }
}

// grid (decode tokens, nh), 64 threads: merges the splits of one (token, head) in ascending order.
// EARLY > 0 (at most that many splits, the usual case): every partial output this lane will need is asked for at
// once, before the weights are worked out: one trip to memory instead of one after the other.  The sums are the same,
// in the same order.
#define MAX_SPLITS 256
template <int EARLY>
__global__ __launch_bounds__(64) void attn_decode_combine_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const float* __restrict__ part_o,
    const float* __restrict__ part_ml, const int4* __restrict__ decode_info, int nh, int num_splits) {
  __shared__ float w_s[MAX_SPLITS];
  const int ti = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int64_t base = ((int64_t)ti * nh + head) * num_splits;
  constexpr int DPL = (HD + 63) / 64;
  float o[DPL][EARLY > 0 ? EARLY : 1];
  const int row = decode_info[ti].x;
  if (EARLY > 0) {
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = lane + 64 * i < HD ? lane + 64 * i : 0;
#pragma unroll
      for (int s = 0; s < EARLY; ++s) o[i][s] = part_o[(base + (s < num_splits ? s : 0)) * HD + d];
    }
  }
  float mx = -INFINITY;
  for (int s = lane; s < num_splits; s += 64) mx = fmaxf(mx, part_ml[(base + s) * 2]);
  mx = wave_max(mx);
  float total = 0.f;
  for (int s = lane; s < num_splits; s += 64) {
    const float ms = part_ml[(base + s) * 2];
    const float w = ms == -INFINITY ? 0.f : fast_exp2(ms - mx);
    w_s[s] = w;
    total += w * part_ml[(base + s) * 2 + 1];
  }
  total = wave_sum(total);
  __syncthreads();
  const float inv = 1.f / total;
  bf16_t* op = out + (int64_t)row * out_stride + (int64_t)head * HD;
  if (EARLY > 0) {
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = lane + 64 * i;
      float acc = 0.f;
#pragma unroll
      for (int s = 0; s < EARLY; ++s)
        if (s < num_splits) acc += o[i][s] * w_s[s];
      if (d < HD) op[d] = f32_to_bf16(acc * inv);
    }
    return;
  }
  for (int d = lane; d < HD; d += 64) {
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < num_splits; ++s) acc += part_o[(base + s) * HD + d] * w_s[s];
    op[d] = f32_to_bf16(acc * inv);
  }
}

// ----------------------------------------------------------------------------- prefill
// Where a tile's keys are dealt to several workgroups (a short prompt makes too few tiles to go round, and its last
// tiles see many times the keys of its first): parts[tile] = (first key, end of keys: multiples of 32, index of the
// tile's first row among the rows whose results come in parts, part + (number of parts << 16)).  Such a workgroup
// leaves its rows unnormalised, with their maxima and sums, where the kernel that merges the splits of single tokens
// finds them: part_o [rows in parts][nh][parts][HD], part_ml [..][2].
struct KeyPart {
  int begin, end, first_row, part, parts;
};
__device__ __forceinline__ KeyPart key_part(const int32_t* __restrict__ parts, int bx, int begin, int end) {
  KeyPart kp = {begin, end, -1, 0, 1};
  if (parts) {
    const int32_t* p = parts + (int64_t)bx * 4;
    const int n = __builtin_amdgcn_readfirstlane(p[3]) >> 16;
    if (n > 1) {
      kp.begin = __builtin_amdgcn_readfirstlane(p[0]);
      kp.end = __builtin_amdgcn_readfirstlane(p[1]);
      kp.first_row = __builtin_amdgcn_readfirstlane(p[2]);
      kp.part = __builtin_amdgcn_readfirstlane(p[3]) & 0xffff;
      kp.parts = n;
    }
  }
  return kp;
}

// The rows of a prefill wavefront, merged over its workgroup's streams: normalised into `out`, or (a tile whose keys
// are in parts) as they are, with maxima and sums, into the workspace.
template <int NB>
__device__ __forceinline__ void write_rows(const f32x4 (&o)[NB][DB], const float (&m)[NB], const float (&l)[NB],
                                           bf16_t* __restrict__ out, int64_t out_stride, float* __restrict__ part_o,
                                           float* __restrict__ part_ml, const KeyPart& kp, int row0, int rows, int head,
                                           int nh, int c, int g) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int j = nb * 16 + c;
    if (j >= rows) continue;
    if (kp.first_row >= 0) {
      const int64_t slot = ((int64_t)(kp.first_row + j) * nh + head) * kp.parts + kp.part;
      float* op = part_o + slot * HD + g * 4;
#pragma unroll
      for (int db = 0; db < DB; ++db) *reinterpret_cast<f32x4*>(op + db * 16) = o[nb][db];
      if (g == 0) {
        part_ml[slot * 2] = m[nb];
        part_ml[slot * 2 + 1] = l[nb];
      }
      continue;
    }
    const float inv = 1.f / l[nb];
    bf16_t* op = out + (int64_t)(row0 + j) * out_stride + (int64_t)head * HD + g * 4;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      union { uint2 u; bf16_t e[4]; } pk;
#pragma unroll
      for (int i = 0; i < 4; ++i) pk.e[i] = f32_to_bf16(o[nb][db][i] * inv);
      *reinterpret_cast<uint2*>(op + db * 16) = pk.u;
    }
  }
}

// grid (tiles, nkv * head_blocks); a workgroup holds hpw * splits wavefronts: hpw query heads of one kv
// head, and for each head `splits` wavefronts that take the key tiles s, s + splits, ... of the same
// 16*NB rows, so that the longest rows of a causal prompt are not one wavefront's serial work.  The
// states of a head's wavefronts meet in LDS: wavefront 0 of the head merges and writes the rows.
// tiles: int32 [n][4] = (entry, first token row of the step, rows (<= 16*NB), first position).
template <int NB>
__global__ __launch_bounds__(64 * PREFILL_WAVES) void attn_prefill_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles, int nh,
    int nkv, int head_blocks, int hpw, int splits, int ps_shift, int window, float scale,
    const int32_t* __restrict__ parts, float* __restrict__ part_o, float* __restrict__ part_ml) {
  extern __shared__ float lds[];          // [hpw][splits-1][NB] x { o[HD][17], m[16], l[16] }
  constexpr int STATE = HD * 17 + 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  // Workgroups are handed out in the order of their linear number and go to the 8 XCDs in turn, each with an L2 of its
  // own.  They are renumbered with the grid's y (kv head x head block) running fastest, linear = x * extent of y + y
  // (one to one for any extents): the heaviest tiles of every y go out first, so that in a step of more workgroups than
  // the chip holds the long walks do not start last; and where y's extent divides 8 an XCD sees one y only, its L2
  // holding the keys and values of one kv head instead of all of them.
  int by = blockIdx.y, bx = blockIdx.x;
  if (gridDim.y > 1) {
    const int linear = blockIdx.x + blockIdx.y * gridDim.x;
    by = linear % gridDim.y;
    bx = linear / gridDim.y;
  }
  const int kvh = by / head_blocks, hb = by % head_blocks;
  const int group = nh / nkv;
  const int hl = wave / splits, split = wave % splits;
  const bool head_ok = hb * hpw + hl < group;
  const int head = kvh * group + hb * hpw + hl;
  const int32_t* tile = tiles + (int64_t)bx * 4;
  const int entry = tile[0], row0 = tile[1], rows = tile[2], pos0 = tile[3];
  const int kv_min_t = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const KeyPart kp = key_part(parts, bx, (kv_min_t / 32) * 32, ((pos0 + rows - 1) / 32 + 1) * 32);

  f32x4 o[NB][DB];
  float m[NB], l[NB];
  init_state<NB>(o, m, l);
  if (head_ok) {
    bf16x8 qr[NB][KB];
    int cpos[NB], clo[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const int j = nb * 16 + c;
      const bool ok = j < rows;
      cpos[nb] = ok ? pos0 + j : -1;
      clo[nb] = (window > 0 && pos0 + j - window + 1 > 0) ? pos0 + j - window + 1 : 0;
      load_q(qr[nb], ok ? q + (int64_t)(row0 + j) * q_stride + (int64_t)head * HD : nullptr, g);
    }
    const int kv_min = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    const int kv_max = pos0 + rows - 1;
    // every row of the tile sees the keys from the last row's window start up to the first row's position
    const int full_lo = (window > 0 && kv_max - window + 1 > 0) ? kv_max - window + 1 : 0;
    attend_tiles<NB, PREFILL_DEPTH>(o, m, l, qr, cpos, clo, k_pages, v_pages,
                                    block_table + (int64_t)__builtin_amdgcn_readfirstlane(entry) * table_width,
                                    table_width, kvh, nkv, ps_shift, kv_min, kv_max, full_lo, pos0,
                                    kp.begin + 32 * split, kp.end, 32 * splits, scale);
    finish_sums<NB>(l);
  }
  if (splits > 1) {
    if (head_ok && split > 0) {
      float* st = lds + (int64_t)((hl * (splits - 1) + split - 1) * NB) * STATE;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        float* sn = st + nb * STATE;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) sn[(db * 16 + g * 4 + i) * 17 + c] = o[nb][db][i];
        if (g == 0) {
          sn[HD * 17 + c] = m[nb];
          sn[HD * 17 + 16 + c] = l[nb];
        }
      }
    }
    __syncthreads();
    if (!head_ok || split > 0) return;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float mx = m[nb];
      for (int sp = 1; sp < splits; ++sp)
        mx = fmaxf(mx, lds[(int64_t)((hl * (splits - 1) + sp - 1) * NB + nb) * STATE + HD * 17 + c]);
      const float f0 = m[nb] == -INFINITY ? 0.f : fast_exp2(m[nb] - mx);
      l[nb] *= f0;
#pragma unroll
      for (int db = 0; db < DB; ++db) o[nb][db] *= f0;
      for (int sp = 1; sp < splits; ++sp) {      // in split order
        const float* sn = lds + (int64_t)((hl * (splits - 1) + sp - 1) * NB + nb) * STATE;
        const float ms = sn[HD * 17 + c];
        const float f = ms == -INFINITY ? 0.f : fast_exp2(ms - mx);
        l[nb] += sn[HD * 17 + 16 + c] * f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[nb][db][i] += sn[(db * 16 + g * 4 + i) * 17 + c] * f;
      }
      m[nb] = mx;                              // what sums and outputs are relative to now (a tile in parts hands it on)
    }
  } else if (!head_ok) {
    return;
  }
  write_rows<NB>(o, m, l, out, out_stride, part_o, part_ml, kp, row0, rows, head, nh, c, g);
}

// ----------------------------------------------------------------------------- prefill, operands through LDS
// For head sizes of 64, 128 and 256.  The wavefronts of a workgroup that attend the same rows to the same key
// tiles (the heads of a kv group, side by side) take their K and V operands from LDS, where ONE further
// wavefront per stream of tiles, the producer, has put them with loads that go from global memory straight
// into LDS.  What this saves is the vector memory unit's time, which is what the register kernel above waits
// for (its time follows the number of tile visits of its wavefronts, whatever each visit computes): a load
// instruction there brings 16 rows of 64 bytes, half a cache line each, once per head; here every instruction
// brings whole lines, once per workgroup, and the heads read LDS.
//   ring: per stream STAGES stages of a tile's keys (32 * HD * 2 bytes) followed by its values (as many).
//   keys of a stage: 16-byte piece `ch` of key row r lies at piece r * CPR + (ch ^ (swz(r) mod CPR)), CPR = HD / 8
//     pieces to a row and swz(r) = 4 * (r / 8) + r % 4: the 16 rows that one matrix-core operand takes, 8 lanes to a
//     clock, then fall into different banks.  Values: piece g (8 keys) of dim d at piece d * 4 + g: an operand is
//     1 KB in a row.
//   every iteration: the producer waits for the loads of the tile the consumers are about to read, all meet at a
//   barrier, the producer issues the loads of the tile STAGES - 1 further on into the stage that was read last.
#if HEAD_DIM == 64 || HEAD_DIM == 128 || HEAD_DIM == 256
#define HAVE_PREFILL_SHARED 1
constexpr int CPR = HD / 8;
constexpr int TILE_K_BYTES = 32 * HD * 2;
constexpr int STAGE_BYTES = 2 * TILE_K_BYTES;
typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void global_void_t;

__device__ __forceinline__ int swz(int r) { return ((r >> 3) << 2) | (r & 3); }

template <int N>
__device__ __forceinline__ void wait_vector_loads_but() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// The producer's loads of one tile.  p0..p3: the pages of the tile (scalars; 0 for a page with no live key).
__device__ __forceinline__ void produce_tile(unsigned char* stage, const bf16_t* __restrict__ k_pages,
                                             const bf16_t* __restrict__ v_pages, int p0, int p1, int p2, int p3,
                                             int kvh, int nkv, int ps_shift, int k0, int lane) {
  const int ps = 1 << ps_shift;
  const int in_page = k0 & (ps - 1);                 // not 0 only where a page holds several tiles
  // keys: instruction i brings the pieces i * 64 .. + 63 of the stage: 64 / CPR whole rows, all of one page
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int piece = i * 64 + lane, r = piece / CPR, ch = (piece % CPR) ^ (swz(r) & (CPR - 1));
    const int which = (i * (64 / CPR)) >> ps_shift;
    const int page = which == 0 ? p0 : which == 1 ? p1 : which == 2 ? p2 : p3;
    const int64_t row = (((int64_t)page * nkv + kvh) << ps_shift) + in_page + (r & (ps - 1));
    __builtin_amdgcn_global_load_lds((global_void_t*)(k_pages + row * HD + ch * 8), (lds_void_t*)(stage + i * 1024), 16,
                                     0, 0);
  }
  // values: instruction i brings dims 16 i .. + 15, four pieces of 8 keys each
  const int d = lane >> 2, piece_keys = (lane & 3) * 8, which = piece_keys >> ps_shift;
  int q0 = p0, q1 = p1, q2 = p2, q3 = p3;           // pinned as values: see pick_page
  asm("" : "+s"(q0));
  asm("" : "+s"(q1));
  asm("" : "+s"(q2));
  asm("" : "+s"(q3));
  int page = q0;
  page = which == 1 ? q1 : page;
  page = which == 2 ? q2 : page;
  page = which == 3 ? q3 : page;
  const int64_t head = ((int64_t)page * nkv + kvh) * HD;
  const int slot = in_page + (piece_keys & (ps - 1));
#pragma unroll
  for (int i = 0; i < DB; ++i)
    __builtin_amdgcn_global_load_lds((global_void_t*)(v_pages + ((head + 16 * i + d) << ps_shift) + slot),
                                     (lds_void_t*)(stage + TILE_K_BYTES + i * 1024), 16, 0, 0);
}

// grid (tiles, nkv * head_blocks); a workgroup holds hpw * splits consumers (hpw heads, each head's keys dealt
// to `splits` wavefronts as in the kernel above) and after them `splits` producers, one per stream of tiles.
template <int NB, int STAGES>
__global__ __launch_bounds__(64 * PREFILL_WAVES) void attn_prefill_shared_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles, int nh,
    int nkv, int head_blocks, int hpw, int splits, int ps_shift, int window, float scale,
    const int32_t* __restrict__ parts, float* __restrict__ part_o, float* __restrict__ part_ml) {
  static_assert(STAGES == 2 || STAGES == 3, "two or three stages");
  extern __shared__ __attribute__((aligned(16))) unsigned char ring[];
  float* lds = reinterpret_cast<float*>(ring);      // after the loop: [hpw][splits-1][NB] x { o[HD][17], m[16], l[16] }
  constexpr int STATE = HD * 17 + 32;
  const int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int by = blockIdx.y, bx = blockIdx.x;             // renumbered as in the kernel above
  if (gridDim.y > 1) {
    const int linear = blockIdx.x + blockIdx.y * gridDim.x;
    by = linear % gridDim.y;
    bx = linear / gridDim.y;
  }
  const int kvh = by / head_blocks, hb = by % head_blocks;
  const int group = nh / nkv;
  const int consumers = hpw * splits;
  const bool producer = wave >= consumers;
  const int stream = producer ? wave - consumers : wave % splits;
  const int hl = producer ? 0 : wave / splits;
  const bool head_ok = !producer && hb * hpw + hl < group;
  const int head = kvh * group + hb * hpw + hl;
  const int32_t* tile = tiles + (int64_t)bx * 4;
  const int entry = __builtin_amdgcn_readfirstlane(tile[0]), row0 = __builtin_amdgcn_readfirstlane(tile[1]),
            rows = __builtin_amdgcn_readfirstlane(tile[2]), pos0 = __builtin_amdgcn_readfirstlane(tile[3]);
  const int kv_min = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int kv_max = pos0 + rows - 1;
  // every row of the tile sees the keys from the last row's window start up to the first row's position
  const int full_lo = (window > 0 && kv_max - window + 1 > 0) ? kv_max - window + 1 : 0;
  const KeyPart kp = key_part(parts, bx, (kv_min / 32) * 32, (kv_max / 32 + 1) * 32);
  const int first = kp.begin, tile_end = kp.end, stride = 32 * splits;
  const int iterations = (tile_end - first + stride - 1) / stride;       // of stream 0, the longest
  const int begin = first + 32 * stream;
  unsigned char* my_ring = ring + (size_t)stream * STAGES * STAGE_BYTES;

  f32x4 o[NB][DB];
  float m[NB], l[NB];
  init_state<NB>(o, m, l);
  if (producer) {
    const int32_t* bt = block_table + (int64_t)entry * table_width;
    const int ps = 1 << ps_shift;
    // the loads of tile number j of the stream, into its stage
    auto produce = [&](int j) {
      const int k0 = begin + j * stride;
      if (k0 >= tile_end) return;
      const int first_page = k0 >> ps_shift;
      int pages[4];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int lo = k0 + (w << ps_shift);                              // the page's first key
        const bool live = (w << ps_shift) < 32 && lo <= kv_max && lo + ps - 1 >= kv_min;
        const int id = table_entry(bt, table_width, first_page + w);
        pages[w] = live ? id : 0;
      }
      produce_tile(my_ring + (j % STAGES) * STAGE_BYTES, k_pages, v_pages, pages[0], pages[1], pages[2], pages[3], kvh,
                   nkv, ps_shift, k0, lane);
    };
#pragma unroll
    for (int j = 0; j < STAGES - 1; ++j) produce(j);
    for (int i = 0; i < iterations; ++i) {
      // tile i is in LDS (a load into LDS counts as done when LDS holds it): what may still be on its way is the
      // tile after it, if the stream has one and the ring a third stage.  No fence here: it would wait for that
      // tile as well.
      if (STAGES == 3 && begin + (i + 1) * stride < tile_end) wait_vector_loads_but<2 * DB>();
      else wait_vector_loads_but<0>();
      __builtin_amdgcn_s_barrier();
      produce(i + STAGES - 1);                             // into the stage that was read in iteration i - 1
    }
  } else {
    bf16x8 qr[NB][KB];
    int cpos[NB], clo[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const int j = nb * 16 + c;
      const bool ok = head_ok && j < rows;
      cpos[nb] = ok ? pos0 + j : -1;
      clo[nb] = (window > 0 && pos0 + j - window + 1 > 0) ? pos0 + j - window + 1 : 0;
      load_q(qr[nb], ok ? q + (int64_t)(row0 + j) * q_stride + (int64_t)head * HD : nullptr, g);
    }
    // where this lane's operands lie in a stage: the two key rows of its products, piece by piece, and its values
    int k_at[2][KB];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int r = 8 * (c >> 2) + 4 * t + (c & 3);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) k_at[t][kb] = (r * CPR + ((kb * 4 + g) ^ (swz(r) & (CPR - 1)))) * 16;
    }
    const int v_at = TILE_K_BYTES + (c * 4 + g) * 16;
    for (int i = 0; i < iterations; ++i) {
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      const int k0 = begin + i * stride;
      if (head_ok && k0 < tile_end) {                      // the same for the whole wavefront
        const unsigned char* stage = my_ring + (i % STAGES) * STAGE_BYTES;
        bf16x8 kr[2][KB], vr[DB];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) kr[t][kb] = *reinterpret_cast<const bf16x8*>(stage + k_at[t][kb]);
#pragma unroll
        for (int db = 0; db < DB; ++db) vr[db] = *reinterpret_cast<const bf16x8*>(stage + v_at + db * 1024);
        f32x4 s[NB][2];
        tile_scores<NB>(s, kr, qr);
        bf16x8 pb[NB];
        tile_softmax<NB>(pb, s, o, m, l, cpos, clo, full_lo, pos0, k0, scale, g);
        tile_output<NB>(o, vr, pb, kv_min, kv_max, k0, g);
      }
    }
    if (head_ok) finish_sums<NB>(l);
  }
  // the wavefronts of a head meet as in the kernel above; first everybody is through with the ring
  __syncthreads();
  const int split = stream;
  if (splits > 1) {
    if (head_ok && split > 0) {
      float* st = lds + (int64_t)((hl * (splits - 1) + split - 1) * NB) * STATE;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        float* sn = st + nb * STATE;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) sn[(db * 16 + g * 4 + i) * 17 + c] = o[nb][db][i];
        if (g == 0) {
          sn[HD * 17 + c] = m[nb];
          sn[HD * 17 + 16 + c] = l[nb];
        }
      }
    }
    __syncthreads();
    if (!head_ok || split > 0) return;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float mx = m[nb];
      for (int sp = 1; sp < splits; ++sp)
        mx = fmaxf(mx, lds[(int64_t)((hl * (splits - 1) + sp - 1) * NB + nb) * STATE + HD * 17 + c]);
      const float f0 = m[nb] == -INFINITY ? 0.f : fast_exp2(m[nb] - mx);
      l[nb] *= f0;
#pragma unroll
      for (int db = 0; db < DB; ++db) o[nb][db] *= f0;
      for (int sp = 1; sp < splits; ++sp) {      // in split order
        const float* sn = lds + (int64_t)((hl * (splits - 1) + sp - 1) * NB + nb) * STATE;
        const float ms = sn[HD * 17 + c];
        const float f = ms == -INFINITY ? 0.f : fast_exp2(ms - mx);
        l[nb] += sn[HD * 17 + 16 + c] * f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[nb][db][i] += sn[(db * 16 + g * 4 + i) * 17 + c] * f;
      }
      m[nb] = mx;                              // what sums and outputs are relative to now (a tile in parts hands it on)
    }
  } else if (!head_ok) {
    return;
  }
  write_rows<NB>(o, m, l, out, out_stride, part_o, part_ml, kp, row0, rows, head, nh, c, g);
}
#endif

extern "C" int ga_attn_head_dim() { return HD; }
// rows of a prefill tile: 16 or (head sizes up to 128) 32
extern "C" int ga_attn_prefill_max_tile_rows() { return 16 * PREFILL_NB; }

// Decode tokens: decode_info holds, for every single new token of the step, int32 x 4 = (its row in the
// step, its position, its entry of the block table, unused).  workspace_o must hold
// n_tokens*nh*num_splits*HD floats and workspace_ml n_tokens*nh*num_splits*2.
extern "C" int ga_attn_decode(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                              const void* v_pages, const void* block_table, int table_width,
                              const void* decode_info, int n_tokens, int nh, int nkv, int page_size, int window, float scale,
                              int split_keys, int num_splits, void* workspace_o, void* workspace_ml,
                              hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (nkv <= 0 || nh % nkv) return -1;
  int ps_shift = 0;
  while ((1 << ps_shift) < page_size) ++ps_shift;
  if ((1 << ps_shift) != page_size || page_size < 8) return -2;
  if (split_keys <= 0 || split_keys % 32 || num_splits <= 0) return -3;
  const int group = nh / nkv, head_blocks = (group + 15) / 16;
  if ((int64_t)nkv * head_blocks > 65535) return -4;
  if (num_splits > MAX_SPLITS) return -5;
  dim3 grid(n_tokens, nkv * head_blocks, num_splits);
  hipLaunchKernelGGL(attn_decode_split_kernel, grid, dim3(64 * DEC_WAVES), 0, stream, (bf16_t*)out, out_stride,
                     (float*)workspace_o, (float*)workspace_ml, (const bf16_t*)q, q_stride,
                     (const bf16_t*)k_pages, (const bf16_t*)v_pages, (const int32_t*)block_table, table_width,
                     (const int4*)decode_info, nh, nkv, head_blocks, ps_shift, window, scale * LOG2E, split_keys,
                     num_splits);
  int rc = GA_CHECK_LAUNCH();
  if (rc || num_splits == 1) return rc;
#define COMBINE(EARLY)                                                                                       \
  hipLaunchKernelGGL(attn_decode_combine_kernel<EARLY>, dim3(n_tokens, nh), dim3(64), 0, stream, (bf16_t*)out, \
                     out_stride, (const float*)workspace_o, (const float*)workspace_ml,                        \
                     (const int4*)decode_info, nh, num_splits)
  if (num_splits <= 8) COMBINE(8);
  else if (num_splits <= 16) COMBINE(16);
  else if (num_splits <= 32) COMBINE(32);
  else COMBINE(0);
#undef COMBINE
  return GA_CHECK_LAUNCH();
}

static int attn_prefill_tiles(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                              const void* v_pages, const void* block_table, int table_width, const void* tiles,
                              int n_tiles, int tile_rows, int nh, int nkv, int page_size, int window, float scale,
                              int fill_workgroups, int prefer_workgroups, const void* parts, void* part_o,
                              void* part_ml, hipStream_t stream);

// parts: null, or for every tile int32 x 4 = (first key, end of keys, index of the tile's first row among the rows that
// come in parts, part + (number of parts << 16)); a tile whose keys are dealt to several workgroups stands in `tiles` once
// per part.  part_rows: int32 x 4 per row that comes in parts (its row of the step first), n_part_rows of them, each in
// num_parts parts; part_o: n_part_rows * nh * num_parts * head_dim floats, part_ml: n_part_rows * nh * num_parts * 2.
extern "C" int ga_attn_prefill(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                               const void* k_pages, const void* v_pages, const void* block_table,
                               int table_width, const void* tiles, int n_tiles, int tile_rows, int nh, int nkv,
                               int page_size, int window, float scale, int fill_workgroups, int prefer_workgroups,
                               const void* parts, const void* part_rows, int n_part_rows, int num_parts, void* part_o,
                               void* part_ml, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (nkv <= 0 || nh % nkv) return -1;
  if (parts && (n_part_rows <= 0 || num_parts < 2 || num_parts > 8 || !part_rows || !part_o || !part_ml)) return -8;
  if (!parts) n_part_rows = 0;
  int rc = attn_prefill_tiles(out, out_stride, q, q_stride, k_pages, v_pages, block_table, table_width, tiles, n_tiles,
                              tile_rows, nh, nkv, page_size, window, scale, fill_workgroups, prefer_workgroups, parts, part_o,
                              part_ml, stream);
  if (rc || n_part_rows == 0) return rc;
  hipLaunchKernelGGL(attn_decode_combine_kernel<8>, dim3(n_part_rows, nh), dim3(64), 0, stream, (bf16_t*)out, out_stride,
                     (const float*)part_o, (const float*)part_ml, (const int4*)part_rows, nh, num_parts);
  return GA_CHECK_LAUNCH();
}

static int attn_prefill_tiles(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                              const void* k_pages, const void* v_pages, const void* block_table,
                              int table_width, const void* tiles, int n_tiles, int tile_rows, int nh, int nkv,
                              int page_size, int window, float scale, int fill_workgroups, int prefer_workgroups,
                              const void* parts, void* part_o, void* part_ml, hipStream_t stream) {
  if (tile_rows != 16 && tile_rows != 16 * PREFILL_NB) return -6;
  int ps_shift = 0;
  while ((1 << ps_shift) < page_size) ++ps_shift;
  if ((1 << ps_shift) != page_size || page_size < 8) return -2;
  const int group = nh / nkv;
  const int nb = tile_rows / 16;
#if defined(HAVE_PREFILL_SHARED) && !defined(PREFILL_SHARED_OFF)
  {
    // at least two heads of a group side by side, and tiles enough to fill the chip with such workgroups: the
    // kernel that shares the operands through LDS.  A workgroup's wavefronts: heads x streams of tiles, and a
    // producer for every stream.
    // Among the divisors of the group that still make fill_workgroups workgroups: the largest that makes prefer_workgroups
    // (one and a half rounds of the chip: the workgroups of the second half-round fill in behind the short walks of the
    // first), else the smallest (the most workgroups).  Measured on MI355X, 12 heads in 2 groups of head size 128, one
    // prompt: 2,048 tokens 3 heads side by side (256 workgroups) 40.5 us, 2 (384) 38.1; 4,096 tokens 6 heads (256) 125 us,
    // 3 (512) 82; 8,192 tokens 6 heads (512) 261 us, 3 (1,024) 272.
    int heads = 1;
    for (int d = PREFILL_WAVES - 1; d >= 2; --d)
      if (group % d == 0 && (int64_t)n_tiles * nkv * (group / d) >= fill_workgroups) {
        heads = d;                                                         // ends at the smallest such divisor
        if ((int64_t)n_tiles * nkv * (group / d) >= prefer_workgroups) break;
      }
    if (heads >= 2) {
      int streams = PREFILL_WAVES / (heads + 1), stages = 3;
      const size_t room = 150 * 1024;
      if ((size_t)streams * stages * STAGE_BYTES > room) stages = 2;
      while (streams > 1 && (size_t)streams * stages * STAGE_BYTES > room) --streams;
      const int head_blocks = group / heads;
      if ((int64_t)nkv * head_blocks > 65535) return -4;
      size_t lds = (size_t)streams * stages * STAGE_BYTES;
      const size_t merge = (size_t)heads * (streams - 1) * nb * (HD * 17 + 32) * sizeof(float);
      if (merge > lds) lds = merge;
      dim3 grid(n_tiles, nkv * head_blocks), block(64 * (heads + 1) * streams);
#define LAUNCH_SHARED(NB, ST)                                                                                  \
  do {                                                                                                         \
    const void* fn = (const void*)attn_prefill_shared_kernel<NB, ST>;                                          \
    if (lds > 48 * 1024 &&                                                                                     \
        hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)           \
      return -7;                                                                                               \
    hipLaunchKernelGGL((attn_prefill_shared_kernel<NB, ST>), grid, block, lds, stream, (bf16_t*)out,           \
                       out_stride, (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, \
                       (const int32_t*)block_table, table_width, (const int32_t*)tiles, nh, nkv, head_blocks,  \
                       heads, streams, ps_shift, window, scale * LOG2E, (const int32_t*)parts, (float*)part_o, \
                       (float*)part_ml);                                                                       \
  } while (0)
      if (nb == 1) {
        if (stages == 3) LAUNCH_SHARED(1, 3); else LAUNCH_SHARED(1, 2);
      } else {
        if (stages == 3) LAUNCH_SHARED(PREFILL_NB, 3); else LAUNCH_SHARED(PREFILL_NB, 2);
      }
#undef LAUNCH_SHARED
      return GA_CHECK_LAUNCH();
    }
  }
#endif
  // heads of a group that share a workgroup, and so the keys they stream: the largest divisor of the group that a
  // workgroup has wavefronts for, smaller where the step has too few tiles to fill the chip, which leaves more
  // wavefronts of a workgroup to split the keys of each head.  Measured on MI355X: 7 heads of a group side by side
  // take 138 us for a 2k-token prompt of 28 heads in 4 groups where one head with its keys split eight ways takes
  // 178; 6 heads side by side 491 us for 8k tokens of 12 heads in 2 groups where 3 heads split two ways take 500
  int hpw = 1;
  for (int d = 2; d <= PREFILL_WAVES; ++d)
    if (group % d == 0 && (int64_t)n_tiles * nkv * (group / d) >= fill_workgroups) hpw = d;
  int splits = PREFILL_WAVES / hpw;
  if (hpw > 1 && splits > 4) splits = 4;
  const int head_blocks = group / hpw;
  if ((int64_t)nkv * head_blocks > 65535) return -4;
  const size_t lds = (size_t)hpw * (splits - 1) * nb * (HD * 17 + 32) * sizeof(float);
  dim3 grid(n_tiles, nkv * head_blocks), block(64 * hpw * splits);
#define LAUNCH(NB)                                                                                        \
  hipLaunchKernelGGL(attn_prefill_kernel<NB>, grid, block, lds, stream, (bf16_t*)out, out_stride,         \
                     (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,           \
                     (const int32_t*)block_table, table_width, (const int32_t*)tiles, nh, nkv, head_blocks, \
                     hpw, splits, ps_shift, window, scale * LOG2E, (const int32_t*)parts, (float*)part_o,   \
                     (float*)part_ml)
  if (lds > 48 * 1024) {                     // more dynamic LDS than the default limit: ask for it
    const void* fn = nb == 1 ? (const void*)attn_prefill_kernel<1> : (const void*)attn_prefill_kernel<PREFILL_NB>;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return -7;
  }
  if (nb == 1) LAUNCH(1); else LAUNCH(PREFILL_NB);
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
