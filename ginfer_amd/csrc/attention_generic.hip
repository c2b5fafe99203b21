// Paged attention, the general kernels: any mix of prompt portions and single decoded tokens, any
// head size up to 256, full or windowed, 32-bit or bfloat16 storage with
// 32-bit scores, softmax and accumulators.  They are the whole of the 32-bit path and the fallback of
// the bfloat16 path.  Three kernels that give the same bits: a wavefront per (token, query head), described first, for
// every size; and two on the matrix cores' 32-bit instruction (further down), at head sizes in steps of 16 up to 128:
// one for the prompt portions of a step, one for its single tokens.
//
// One wavefront per (token, query head).  A token is self-describing: `token_entry[t]` names its
// row of the block table and `positions[t]` its absolute position p, so it attends to the keys
// c in [max(0, p - window + 1), p] of its own request (all keys c <= p when window == 0): the
// reference's mask `c <= r + (kv_len - q_len) && c < kv_len`
// (ginfer/core/op/kernels/cuda/page_attn_kernel/flash_gqa_varlen_kernel.cu:202-222) in absolute
// positions.  score = (q . k) * scale with the scale applied to the 32-bit dot product; online
// softmax over key tiles of 64 (:474-499), here with tiles fixed at absolute multiples of 64 and
// every reduction in a fixed order, so a token's result is bit-identical however the request was
// cut into steps, whatever else is in the batch and wherever its pages lie.  Head h reads kv head
// h / (nh / nkv) (:439-450).  Keys are fetched through block_table[entry][c / page_size].
//
// A workgroup holds the wavefronts of `tq` neighbouring tokens of the step and of all query heads of ONE kv head.
// Tokens of the same request see the same keys, and so do the heads of a kv group: a tile of 64 keys and their values
// comes from the pages ONCE per workgroup, with consecutive lanes on consecutive elements, into LDS (keys [key][dim],
// values [dim][key], each row padded by four words so that rows stay 16-byte aligned and neither a lane per key nor a
// lane per dimension meets a bank twice), and every wavefront takes its operands from there.  What a wavefront computes, and in which order it adds,
// does not depend on what shares the workgroup with it: its dot products run over the dimensions in ascending order,
// its sums over the keys of a tile likewise, and tiles follow each other in ascending order.
#include <type_traits>

#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

#define MAX_HD 256
#define GA_MAX_WAVES 16
#define KPAD 4              // floats that pad a row of keys in LDS: rows stay 16-byte aligned, lanes on different banks
#define VS (WAVE + 4)       // a row of values in LDS, in floats

// VEC elements (16 bytes) of T per load where head size and page size allow it, else one
template <typename T, int VEC>
struct VecLoad {
  float v[VEC];
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = 0.f;
  }
  __device__ __forceinline__ void load(const T* p) {
    if (VEC == 1) {
      v[0] = Num<T>::ld(p);
    } else {
      const uint4 raw = *reinterpret_cast<const uint4*>(p);
      const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = Num<T>::ld(e + i);
    }
  }
};

#define GA_BATCH 4         // loads of keys, and as many of values, that a thread has under way at a time

// Whether the tokens around token t that are of its request (neighbours in the step: a request's tokens lie side by
// side) are fewer than n.  The two kernels below share a step by this: runs of at least MA_MIN_RUN tokens go to the
// matrix cores, shorter ones (the single tokens of decoding requests beside a prompt portion, which each walk the keys
// of another request) to a wavefront per token and head.
__device__ __forceinline__ bool run_is_shorter(const int32_t* __restrict__ token_entry, int64_t t, int tokens, int n) {
  const int e = token_entry[t];
  int len = 1;
  for (int i = 1; len < n && t - i >= 0 && token_entry[t - i] == e; ++i) ++len;
  for (int i = 1; len < n && t + i < tokens && token_entry[t + i] == e; ++i) ++len;
  return len < n;
}

// PIPE: the wavefronts beyond those that compute are loaders: they bring tile i + 1 into a second buffer while the
// others multiply tile i, one barrier a tile (the launcher says when: few workgroups, both buffers fit, and at least
// as many wavefronts load as compute).
template <typename T, int VEC, bool PIPE>
__global__ __launch_bounds__(64 * GA_MAX_WAVES) void paged_attention_generic_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ token_entry, const int32_t* __restrict__ positions, int tokens, int nh, int nkv,
    int hd, int page_size, int window, float scale, int tq, int hpw, int min_run) {
  extern __shared__ float lds[];
  const int group = nh / nkv, head_blocks = (group + hpw - 1) / hpw;     // hpw heads of a kv group to a workgroup
  const int waves = tq * hpw, threads = blockDim.x;        // wavefronts that compute; all threads load (see the launcher)
  const int ks = hd + KPAD;                      // a key's row in LDS, in floats
  const int tile_floats = WAVE * ks + hd * VS;    // a tile in LDS: keys [64][hd + KPAD], then values [hd][64 + 4]
  constexpr int nbuf = PIPE ? 2 : 1;
  float* q_s = lds + nbuf * tile_floats;         // [waves][hd]
  float* p_s = q_s + waves * hd;                 // [waves][64]
  int32_t* page_s = reinterpret_cast<int32_t*>(p_s + waves * WAVE);     // [nbuf][64]: the page of every key of a tile, or -1
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int g = blockIdx.y / head_blocks, hl = (blockIdx.y % head_blocks) * hpw + wave % hpw;
  const int tl = wave / hpw, h = g * group + hl;                  // the wavefront's token of the workgroup, and head
  const int64_t t0 = (int64_t)blockIdx.x * tq;
  const int64_t t = t0 + tl;
  const bool live = wave < waves && t < tokens && hl < group;
  const int pos = live ? positions[t] : -1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  if (live) {
    const T* qp = q + t * q_stride + (int64_t)h * hd;
    for (int d = lane; d < hd; d += WAVE) q_s[wave * hd + d] = Num<T>::ld(qp + d);
  }

  float m = -INFINITY, l = 0.f;
  float acc[MAX_HD / WAVE];
#pragma unroll
  for (int i = 0; i < MAX_HD / WAVE; ++i) acc[i] = 0.f;
  bool done = false;           // this wavefront's token was of a run that this kernel handles

  // The workgroup's tokens fall into runs of one request each (a prompt portion: one run; single tokens of several
  // requests: a run each).  A run's tiles are loaded once and serve every wavefront of the run.
  int run_begin = 0;
  while (run_begin < tq && t0 + run_begin < tokens) {
    const int run_entry = token_entry[t0 + run_begin];
    int run_end = run_begin, lo_min = 0x7fffffff, pos_max = -1;
    while (run_end < tq && t0 + run_end < tokens && token_entry[t0 + run_end] == run_entry) {
      const int p = positions[t0 + run_end];
      const int l0 = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
      lo_min = l0 < lo_min ? l0 : lo_min;
      pos_max = p > pos_max ? p : pos_max;
      ++run_end;
    }
    // min_run > 0: runs of that many tokens and more are the other kernel's
    if (min_run > 0 && !run_is_shorter(token_entry, t0 + run_begin, tokens, min_run)) {
      run_begin = run_end;
      continue;
    }
    const bool mine = live && tl >= run_begin && tl < run_end;
    done = done || mine;
    const int32_t* bt = block_table + (int64_t)run_entry * table_width;
    const int first_page = lo_min / page_size, last_page = pos_max / page_size;    // the pages that the run reads
    // the page of every key of a tile, asked for one tile ahead
    auto tile_page = [&](int tile) -> int32_t {
      if (threadIdx.x >= WAVE || tile > pos_max) return -1;
      const int pi = (tile + (int)threadIdx.x) / page_size;
      return (pi >= first_page && pi <= last_page) ? bt[pi] : -1;
    };
    const int per_key = hd / VEC, per_dim = WAVE / VEC, nvec = WAVE * per_key;       // as many vectors of values as of keys
    // keys: VEC dimensions of one key to a load, consecutive threads on consecutive dimensions; values: VEC keys of
    // one dimension to a load (a page keeps the keys of a dimension side by side).  A batch of both is under way
    // before the first of it is put into LDS.
    constexpr int NB = GA_BATCH;
    // the threads that load, and this thread's number among them
    const int loaders = PIPE ? threads - waves * WAVE : threads;
    const int ltid = PIPE ? (int)threadIdx.x - waves * WAVE : (int)threadIdx.x;
    VecLoad<T, VEC> rk[NB], rv[NB];
    bool okk[NB], okv[NB];
    auto ask = [&](int tile, int base, const int32_t* pages) {
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        const int j = v / per_key, d = (v - j * per_key) * VEC;
        const int64_t page = v < nvec ? pages[j] : -1;
        okk[u] = page >= 0;
        if (okk[u]) rk[u].load(k_pages + ((page * nkv + g) * page_size + ((tile + j) % page_size)) * hd + d);
      }
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        const int d = v / per_dim, j = (v - d * per_dim) * VEC;
        const int64_t page = v < nvec ? pages[j] : -1;
        okv[u] = page >= 0;
        if (okv[u]) rv[u].load(v_pages + ((page * nkv + g) * hd + d) * page_size + ((tile + j) % page_size));
      }
    };
    auto put = [&](int base, float* k_s, float* v_s) {
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        const int j = v / per_key, d = (v - j * per_key) * VEC;
        if (okk[u]) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) k_s[j * ks + d + i] = rk[u].v[i];
        }
      }
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        const int d = v / per_dim, j = (v - d * per_dim) * VEC;
        if (okv[u]) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) v_s[d * VS + j + i] = rv[u].v[i];
        }
      }
    };
    // one tile of this wavefront's token, its keys and values in LDS
    auto attend = [&](int tile, const float* k_s, const float* v_s) {
      if (!mine || tile > pos || tile + WAVE - 1 < lo) return;        // not a tile of this wavefront's token
      const int c = tile + lane;
      const bool valid = c >= lo && c <= pos;
      float s = -INFINITY;
      if (valid) {
        const float* kr = k_s + lane * ks;
        const float* qr = q_s + wave * hd;
        float dot = 0.f;
        int d = 0;
        if ((hd & 3) == 0) {                      // four dimensions to an LDS read; the sum keeps its order
          for (; d < hd; d += 4) {
            const float4 qq = *reinterpret_cast<const float4*>(qr + d);
            const float4 kk = *reinterpret_cast<const float4*>(kr + d);
            dot = __builtin_fmaf(qq.x, kk.x, dot);
            dot = __builtin_fmaf(qq.y, kk.y, dot);
            dot = __builtin_fmaf(qq.z, kk.z, dot);
            dot = __builtin_fmaf(qq.w, kk.w, dot);
          }
        }
        for (; d < hd; ++d) dot = __builtin_fmaf(qr[d], kr[d], dot);
        s = dot * scale;
      }
      const float m_new = fmaxf(m, wave_max(s));   // finite: every tile holds at least one valid key
      const float p = valid ? expf(s - m_new) : 0.f;
      const float alpha = expf(m - m_new);         // exp(-inf) = 0 on the first tile
      l = __builtin_fmaf(l, alpha, wave_sum(p));
      m = m_new;
      p_s[wave * WAVE + lane] = p;                 // read by this wavefront alone: LDS keeps a wavefront's order
      __builtin_amdgcn_wave_barrier();
      const int j0 = lo > tile ? lo - tile : 0;
      const int j1 = pos - tile < WAVE - 1 ? pos - tile : WAVE - 1;
      const float* pr = p_s + wave * WAVE;
#pragma unroll
      for (int i = 0; i < MAX_HD / WAVE; ++i) {
        const int d = lane + i * WAVE;
        if (d < hd) {
          const float* vr = v_s + d * VS;
          float a = acc[i] * alpha;
          int j = j0;
          for (; j <= j1 && (j & 3); ++j) a = __builtin_fmaf(pr[j], vr[j], a);
          for (; j + 3 <= j1; j += 4) {            // four keys to an LDS read, added in ascending order
            const float4 pp = *reinterpret_cast<const float4*>(pr + j);
            const float4 vv = *reinterpret_cast<const float4*>(vr + j);
            a = __builtin_fmaf(pp.x, vv.x, a);
            a = __builtin_fmaf(pp.y, vv.y, a);
            a = __builtin_fmaf(pp.z, vv.z, a);
            a = __builtin_fmaf(pp.w, vv.w, a);
          }
          for (; j <= j1; ++j) a = __builtin_fmaf(pr[j], vr[j], a);
          acc[i] = a;
        }
      }
      __builtin_amdgcn_wave_barrier();
    };
    const int first_tile = (lo_min / WAVE) * WAVE;
    if (!PIPE) {
      int32_t my_page = tile_page(first_tile);
      float* k_s = lds;
      float* v_s = lds + WAVE * ks;
      for (int tile = first_tile; tile <= pos_max; tile += WAVE) {
        __syncthreads();                            // the tile before has been read (and q_s is written)
        if (threadIdx.x < WAVE) page_s[threadIdx.x] = my_page;
        __syncthreads();
        my_page = tile_page(tile + WAVE);           // on its way while this tile is loaded and multiplied
        for (int base = threadIdx.x; base < nvec; base += threads * GA_BATCH) {
          ask(tile, base, page_s);
          put(base, k_s, v_s);
        }
        __syncthreads();
        attend(tile, k_s, v_s);
      }
    } else {
      // The pages of a tile are looked up two tiles ahead (by the first wavefront, which computes); the loaders put
      // tile i + 1 into the buffer that tile i - 1 was read from.
      const bool loader = wave >= waves;
      __syncthreads();                              // the run before has been read (and q_s is written)
      if (threadIdx.x < WAVE) page_s[threadIdx.x] = tile_page(first_tile);
      __syncthreads();
      if (loader) {
        for (int base = ltid; base < nvec; base += loaders * GA_BATCH) {
          ask(first_tile, base, page_s);
          put(base, lds, lds + WAVE * ks);
        }
      }
      if (threadIdx.x < WAVE) page_s[WAVE + threadIdx.x] = tile_page(first_tile + WAVE);
      __syncthreads();
      int b = 0;
      for (int tile = first_tile; tile <= pos_max; tile += WAVE, b ^= 1) {
        if (loader) {
          if (tile + WAVE <= pos_max) {
            for (int base = ltid; base < nvec; base += loaders * GA_BATCH) {
              ask(tile + WAVE, base, page_s + (b ^ 1) * WAVE);
              put(base, lds + (b ^ 1) * tile_floats, lds + (b ^ 1) * tile_floats + WAVE * ks);
            }
          }
        } else {
          const int32_t my_page = tile_page(tile + 2 * WAVE);
          attend(tile, lds + b * tile_floats, lds + b * tile_floats + WAVE * ks);
          if (threadIdx.x < WAVE) page_s[b * WAVE + threadIdx.x] = my_page;   // read again two tiles on
        }
        __syncthreads();
      }
    }
    run_begin = run_end;
  }
  if (!done) return;
  T* op = out + t * out_stride + (int64_t)h * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < MAX_HD / WAVE; ++i) {
    const int d = lane + i * WAVE;
    if (d < hd) Num<T>::st(op + d, acc[i] * inv);
  }
}

// What the loading wavefronts of the matrix-core kernels do for one run of tokens: tiles of 64 keys and their values
// from the pages into one of two buffers in LDS.  A row of keys in LDS holds dimension d at (d % 4) * (HD / 4) + d / 4,
// a row of values key j at (j % 4) * 16 + j / 4: lane (row, kq) of a matrix operand wants every fourth element from
// kq on, and so reads four of them at a time; the rows' padding puts the 16 rows of a read on different banks.
template <typename T, int VEC, int HD, int NLOAD>
struct TileLoader {
  static constexpr int KS = HD + KPAD;
  static constexpr int tile_floats = WAVE * KS + HD * VS;
  static constexpr int per_key = HD / VEC, per_dim = WAVE / VEC, nvec = WAVE * per_key;
  static constexpr int NB = VEC == 1 ? 8 : 4;       // loads of keys, and as many of values, under way in a thread
  static constexpr int loaders = NLOAD * WAVE;
  static constexpr bool whole_rounds = nvec % (loaders * NB) == 0;
  const T* k_pages;
  const T* v_pages;
  const int32_t* bt;           // the request's row of the block table
  int nkv, g, page_size, lo_min, pos_max, ltid;
  float* lds;                  // two tile buffers
  int64_t* base_s;             // [2][64]
  int32_t* plain_s;            // [2]

  // where the page of key `tile + ltid` begins for this kv head, in elements (both caches keep page_size * HD
  // elements per page and kv head), or -1 for a key without a page; by the first loading wavefront
  __device__ __forceinline__ int64_t tile_base(int tile) const {
    if (tile > pos_max) return -1;
    const int pi = (tile + ltid) / page_size;
    if (pi < lo_min / page_size || pi > pos_max / page_size) return -1;
    const int64_t page = bt[pi];
    return page >= 0 ? (page * nkv + g) * page_size * HD : -1;
  }
  // a tile into a buffer: all its loads of a round are under way before the first is put into LDS; what lies
  // outside the run's keys, or has no page, becomes zero (what lies in a page beyond a request's last key may be
  // anything, and zero times it must be zero).  PLAIN: every key of the tile has a page and is one of the run's:
  // nothing to ask.
  template <bool PLAIN>
  __device__ __forceinline__ void load_tile(int tile, const int64_t* bases, float* k_s, float* v_s) const {
    for (int base = ltid; base < nvec; base += loaders * NB) {
      VecLoad<T, VEC> rk[NB], rv[NB];
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        const int j = v / per_key, d = (v - j * per_key) * VEC;
        // with 16-byte loads a page's size divides 64, and a tile begins where a page does
        const int in_page = VEC > 1 ? (j & (page_size - 1)) : (tile + j) % page_size;
        if (PLAIN) {
          if (whole_rounds || v < nvec) rk[u].load(k_pages + bases[j] + in_page * HD + d);
        } else {
          const int64_t at = v < nvec ? bases[j] : -1;
          rk[u].zero();
          if (at >= 0 && tile + j >= lo_min && tile + j <= pos_max) rk[u].load(k_pages + at + in_page * HD + d);
        }
      }
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        const int d = v / per_dim, j = (v - d * per_dim) * VEC;
        const int in_page = VEC > 1 ? (j & (page_size - 1)) : (tile + j) % page_size;
        if (PLAIN) {
          if (whole_rounds || v < nvec) rv[u].load(v_pages + bases[j] + d * page_size + in_page);
        } else {
          const int64_t at = v < nvec ? bases[j] : -1;
          rv[u].zero();
          if (at >= 0) rv[u].load(v_pages + at + d * page_size + in_page);
        }
      }
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        if (!whole_rounds && v >= nvec) continue;
        const int j = v / per_key, d = (v - j * per_key) * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i) k_s[j * KS + ((d + i) & 3) * (HD / 4) + ((d + i) >> 2)] = rk[u].v[i];
      }
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const int v = base + u * loaders;
        if (!whole_rounds && v >= nvec) continue;
        const int d = v / per_dim, j = (v - d * per_dim) * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const int c = tile + j + i;
          const bool out_of_range = !PLAIN && (c < lo_min || c > pos_max);
          v_s[d * VS + ((j + i) & 3) * (WAVE / 4) + ((j + i) >> 2)] = out_of_range ? 0.f : rv[u].v[i];
        }
      }
    }
  }
  // a tile's bases into LDS, and whether the tile is plain
  __device__ __forceinline__ void note_tile(int tile, int slot) const {
    if (ltid >= WAVE) return;
    const int64_t at = tile_base(tile);
    base_s[slot * WAVE + ltid] = at;
    const bool plain = __ballot(at >= 0) == ~0ull && tile >= lo_min && tile + WAVE - 1 <= pos_max;
    if (ltid == 0) plain_s[slot] = plain ? 1 : 0;
  }
  __device__ __forceinline__ void load(int tile, int slot) const {
    float* buf = lds + slot * tile_floats;
    if (plain_s[slot]) load_tile<true>(tile, base_s + slot * WAVE, buf, buf + WAVE * KS);
    else load_tile<false>(tile, base_s + slot * WAVE, buf, buf + WAVE * KS);
  }
  // The run's tiles one after the other, tile i + 1 into the buffer that tile i - 1 was read from while the others
  // multiply tile i: `barriers` barriers a tile, which the wavefronts that multiply meet as well (three before the
  // first tile).
  __device__ __forceinline__ void run(int barriers) const {
    const int first_tile = (lo_min / WAVE) * WAVE;
    __syncthreads();                              // the run before has been read
    note_tile(first_tile, 0);
    __syncthreads();
    load(first_tile, 0);
    note_tile(first_tile + WAVE, 1);
    __syncthreads();
    int b = 0;
    for (int tile = first_tile; tile <= pos_max; tile += WAVE, b ^= 1) {
      if (tile + WAVE <= pos_max) load(tile + WAVE, b ^ 1);
      note_tile(tile + 2 * WAVE, b);               // read two tiles on
      for (int i = 0; i < barriers; ++i) __syncthreads();
    }
  }
};

// The same attention on the matrix cores, for steps that hold prompt portions.  v_mfma_f32_16x16x4_f32 takes 32-bit
// operands and adds its four products into the accumulator in ascending k as fused multiply-adds, so a score is the
// chain over ascending dimensions, and an output element the chain over ascending keys, that the kernel above computes:
// the same bits (a key that a token does not see enters its chain as a product with zero, which leaves the sum as it
// is; only a sum that is exactly -0 would become +0).  A wavefront holds one head of MA_COLS neighbouring tokens: the
// scores of a tile are [64 keys][16 tokens] in four accumulators, lane (token, kq) holding keys 16 b + 4 kq + r of its
// token, so the maximum and the sum over a tile's keys are taken in registers and two exchanges, the sum in the order
// of the butterfly above: key bits 5, 4, 3, 2, 1, 0.  The probabilities go through LDS, half a tile at a time, to
// become the second operand of the product with the values.  Queries stay in registers.  A workgroup holds `tq`
// groups of MA_COLS tokens and `hpw` heads of one kv head; its tokens fall into runs of one request as above, and a
// token outside the run, or one that sees no key of the tile, keeps its state through the tile: scale one,
// probabilities zero.  Keys and values beyond the run's range are put into LDS as zeros: what lies in a page beyond a
// request's last key may be anything, and zero times it must be zero.  The wavefronts beyond those that compute are
// loaders: they bring tile i + 1 into a second buffer while the others multiply tile i, one barrier a tile.
#define MA_COLS 16
#define MA_MAX_COMPUTE 12
#define MA_LOADERS 4
#define MA_MIN_RUN 8        // shorter runs of tokens are left to the kernel above
typedef __attribute__((ext_vector_type(4))) float f32x4;

template <typename T, int VEC, int HD>
__global__ __launch_bounds__(64 * (MA_MAX_COMPUTE + MA_LOADERS)) void paged_attention_matrix_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ token_entry, const int32_t* __restrict__ positions, int tokens, int nh, int nkv,
    int page_size, int window, float scale, int tq, int hpw) {
  extern __shared__ float lds[];
  constexpr int hd = HD;
  constexpr int KS = HD + KPAD;                  // the layout of a tile in LDS: TileLoader
  constexpr int NBLK = HD / 16;                  // blocks of 16 dimensions of the output
  constexpr int tile_floats = WAVE * KS + HD * VS;
  const int group = nh / nkv, head_blocks = (group + hpw - 1) / hpw;
  const int waves = tq * hpw, span = tq * MA_COLS;          // wavefronts that compute; tokens of the workgroup
  float* p_all = lds + 2 * tile_floats;          // [waves][32][MA_COLS]
  int64_t* base_s = reinterpret_cast<int64_t*>(p_all + waves * (WAVE / 2) * MA_COLS);      // [2][64]
  int32_t* plain_s = reinterpret_cast<int32_t*>(base_s + 2 * WAVE);                        // [2]
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int col = lane & 15, kq = lane >> 4;
  const bool loader = wave >= waves;
  const int ct = wave / hpw;                                      // the wavefront's group of tokens
  // the workgroups of the step's last tokens come first: they have the most keys to walk, and the compute units that
  // finish the short ones early take what is left
  const int ny = nkv * head_blocks, by = blockIdx.x % ny, bx = gridDim.x / ny - 1 - blockIdx.x / ny;
  const int g = by / head_blocks, hl = (by % head_blocks) * hpw + wave % hpw;
  const int h = g * group + hl;
  const int64_t t0 = (int64_t)bx * span;
  const int tl = ct * MA_COLS + col;                              // this lane's token of the workgroup: a column of the scores
  const int64_t t = t0 + tl;
  const bool live = !loader && hl < group && t < tokens;
  const int pos = live ? positions[t] : -1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int ltid = (int)threadIdx.x - waves * WAVE;          // a loading thread's number
  // The workgroup's tokens from `begin` on that are of one request: the run's end, and the range of keys that its
  // tokens see.  Loaders and the others walk the same runs and tiles, and meet at the same barriers.
  struct Run { int entry, end, lo_min, pos_max; bool skipped; };
  auto next_run = [&](int begin) -> Run {
    Run r{token_entry[t0 + begin], begin, 0x7fffffff, -1, run_is_shorter(token_entry, t0 + begin, tokens, MA_MIN_RUN)};
    while (r.end < span && t0 + r.end < tokens && token_entry[t0 + r.end] == r.entry) {
      const int p = positions[t0 + r.end];
      const int l0 = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
      r.lo_min = l0 < r.lo_min ? l0 : r.lo_min;
      r.pos_max = p > r.pos_max ? p : r.pos_max;
      ++r.end;
    }
    return r;
  };

  if (loader) {
    for (int run_begin = 0; run_begin < span && t0 + run_begin < tokens;) {
      const Run run = next_run(run_begin);
      if (run.skipped) {
        run_begin = run.end;
        continue;
      }
      const TileLoader<T, VEC, HD, MA_LOADERS> loading{k_pages, v_pages, block_table + (int64_t)run.entry * table_width,
                                                       nkv, g, page_size, run.lo_min, run.pos_max, ltid, lds, base_s, plain_s};
      loading.run(1);
      run_begin = run.end;
    }
    return;
  }

  float qr[HD / 4];                                    // the token's query at dimensions 4 i + kq
#pragma unroll
  for (int i = 0; i < HD / 4; ++i) qr[i] = 0.f;
  if (live) {
    const T* qp = q + t * q_stride + (int64_t)h * hd + kq;
#pragma unroll
    for (int i = 0; i < HD / 4; ++i) qr[i] = Num<T>::ld(qp + 4 * i);
  }
  float m = -INFINITY, l = 0.f;
  f32x4 acc[NBLK];
#pragma unroll
  for (int i = 0; i < NBLK; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float* p_s = p_all + wave * (WAVE / 2) * MA_COLS;
  bool done = false;           // this lane's token was of a run that this kernel handles
  for (int run_begin = 0; run_begin < span && t0 + run_begin < tokens;) {
    const Run run = next_run(run_begin);
    if (run.skipped) {
      run_begin = run.end;
      continue;
    }
    const bool mine = live && tl >= run_begin && tl < run.end;
    done = done || mine;
    // one tile for this wavefront's tokens, its keys and values in LDS
    auto attend = [&](int tile, const float* k_s, const float* v_s) {
      const bool active = mine && !(tile > pos || tile + WAVE - 1 < lo);
      if (__ballot(active) == 0) return;                 // no token of this wavefront sees the tile
      // scores: block b holds keys 16 b .. 16 b + 15 of the tile; lane (col, kq) gives key col's dimension 4 i + kq
      f32x4 s[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) s[b] = f32x4{0.f, 0.f, 0.f, 0.f};
      const float* ka = k_s + col * KS + kq * (HD / 4);
#pragma unroll
      for (int n = 0; n < HD / 16; ++n) {
        float4 a[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) a[b] = *reinterpret_cast<const float4*>(ka + b * 16 * KS + 4 * n);
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int b = 0; b < 4; ++b)
            s[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(reinterpret_cast<const float*>(&a[b])[e], qr[4 * n + e], s[b], 0, 0, 0);
      }
      // element r of block b: key 16 b + 4 kq + r of the tile, for this lane's token.  Where every token of the
      // wavefront sees all 64 keys (most tiles of a long prompt) nothing needs a mask: the same arithmetic without
      // the selects.
      const bool whole = __ballot(active && tile >= lo && tile + WAVE - 1 <= pos) == ~0ull;
      float m_new, alpha;
      if (whole) {
        float mx = -INFINITY;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            s[b][r] = s[b][r] * scale;
            mx = fmaxf(mx, s[b][r]);
          }
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
        m_new = fmaxf(m, mx);
        alpha = expf(m - m_new);                   // exp(-inf) = 0 on a token's first tile
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) s[b][r] = expf(s[b][r] - m_new);
      } else {
        float mx = -INFINITY;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int c = tile + 16 * b + 4 * kq + r;
            s[b][r] = (active && c >= lo && c <= pos) ? s[b][r] * scale : -INFINITY;
            mx = fmaxf(mx, s[b][r]);
          }
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
        m_new = fmaxf(m, mx);                      // finite for a token that sees the tile: it holds one of its keys
        alpha = active ? expf(m - m_new) : 1.f;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int c = tile + 16 * b + 4 * kq + r;
            s[b][r] = (active && c >= lo && c <= pos) ? expf(s[b][r] - m_new) : 0.f;
          }
        m_new = active ? m_new : m;
      }
      float u[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) u[r] = (s[0][r] + s[2][r]) + (s[1][r] + s[3][r]);     // key bits 5, then 4
#pragma unroll
      for (int r = 0; r < 4; ++r) u[r] = u[r] + __shfl_xor(u[r], 32, WAVE);             // key bit 3
#pragma unroll
      for (int r = 0; r < 4; ++r) u[r] = u[r] + __shfl_xor(u[r], 16, WAVE);             // key bit 2
      const float sum = (u[0] + u[2]) + (u[1] + u[3]);                                  // key bits 1 and 0
      l = __builtin_fmaf(l, alpha, sum);
      m = m_new;
      if (__ballot(alpha != 1.f) != 0) {             // times one changes nothing
#pragma unroll
        for (int i = 0; i < NBLK; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][r] = acc[i][r] * alpha;
      }
      // values: lane (col, kq) gives dimension 16 blk + col at key 4 j + kq, and its token's probability of that key
      const float* va = v_s + col * VS + kq * (WAVE / 4);
      const float* pb = p_s + kq * MA_COLS + col;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) p_s[(16 * b + 4 * kq + r) * MA_COLS + col] = s[2 * hf + b][r];
        __builtin_amdgcn_wave_barrier();             // read by this wavefront alone: LDS keeps a wavefront's order
#pragma unroll
        for (int n = 0; n < 2; ++n) {
          float4 v[NBLK];
#pragma unroll
          for (int i = 0; i < NBLK; ++i) v[i] = *reinterpret_cast<const float4*>(va + i * 16 * VS + 8 * hf + 4 * n);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float pj = pb[4 * (4 * n + e) * MA_COLS];
#pragma unroll
            for (int i = 0; i < NBLK; ++i)
              acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(reinterpret_cast<const float*>(&v[i])[e], pj, acc[i], 0, 0, 0);
          }
        }
        __builtin_amdgcn_wave_barrier();
      }
    };
    const int first_tile = (run.lo_min / WAVE) * WAVE;
    __syncthreads();
    __syncthreads();
    __syncthreads();
    int b = 0;
    for (int tile = first_tile; tile <= run.pos_max; tile += WAVE, b ^= 1) {
      const float* buf = lds + b * tile_floats;
      attend(tile, buf, buf + WAVE * KS);
      __syncthreads();
    }
    run_begin = run.end;
  }
  if (!done) return;
  T* op = out + t * out_stride + (int64_t)h * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < NBLK; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) Num<T>::st(op + i * 16 + 4 * kq + r, acc[i][r] * inv);
}

// Single tokens on the matrix cores: the heads of a kv group are the columns.  A workgroup holds one token and (up to
// 16 heads of) one kv head; the scores of a tile are [64 keys][heads], and the four wavefronts that multiply take 16
// keys each, then, for the product with the values, their share of the output's blocks of 16 dimensions each.  Between
// the two they meet twice: once for the tile's maximum (each gives its 16 keys' maximum per head through LDS), once
// for the probabilities, which all of them read from LDS: as the second operand of their products, and to add up a
// head's 64 of them in the order of the butterfly (key bits 5 to 0), every wavefront for itself.  The keys and values
// of a tile are read from LDS once, not once per head as with a wavefront per head, which is what bounds that kernel.
// Scores, maxima, exponentials, sums and outputs are those of the other two kernels to the bit.
#define HA_COMPUTE 4
#define HA_LOADERS 8

template <typename T, int VEC, int HD>
__global__ __launch_bounds__(64 * (HA_COMPUTE + HA_LOADERS)) void paged_attention_heads_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ token_entry, const int32_t* __restrict__ positions, int tokens, int nh, int nkv,
    int page_size, int window, float scale, int min_run) {
  extern __shared__ float lds[];
  constexpr int KS = HD + KPAD;                  // the layout of a tile in LDS: TileLoader
  constexpr int NBLK = HD / 16;                  // blocks of 16 dimensions of the output
  constexpr int BPW = (NBLK + HA_COMPUTE - 1) / HA_COMPUTE;       // ... of a wavefront: blocks wave, wave + 4, ...
  constexpr int tile_floats = WAVE * KS + HD * VS;
  const int group = nh / nkv, head_blocks = (group + 15) / 16;
  float* p_s = lds + 2 * tile_floats;            // [64 keys][16 heads]
  float* mx_s = p_s + WAVE * 16;                 // [4][16]
  int64_t* base_s = reinterpret_cast<int64_t*>(mx_s + HA_COMPUTE * 16);      // [2][64]
  int32_t* plain_s = reinterpret_cast<int32_t*>(base_s + 2 * WAVE);          // [2]
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int col = lane & 15, kq = lane >> 4;
  const int64_t t = blockIdx.x;
  // min_run > 0: the tokens of runs of that many and more are another kernel's
  if (min_run > 0 && !run_is_shorter(token_entry, t, tokens, min_run)) return;
  const int g = blockIdx.y / head_blocks, hl = (blockIdx.y % head_blocks) * 16 + col;
  const int h = g * group + hl;
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  if (wave >= HA_COMPUTE) {
    const TileLoader<T, VEC, HD, HA_LOADERS> loading{k_pages, v_pages, block_table + (int64_t)token_entry[t] * table_width,
                                                     nkv, g, page_size, lo, pos, (int)threadIdx.x - HA_COMPUTE * WAVE,
                                                     lds, base_s, plain_s};
    loading.run(3);
    return;
  }
  const bool live = hl < group;                  // this lane's column has a head
  float qr[HD / 4];                              // the head's query at dimensions 4 i + kq
#pragma unroll
  for (int i = 0; i < HD / 4; ++i) qr[i] = 0.f;
  if (live) {
    const T* qp = q + t * q_stride + (int64_t)h * HD + kq;
#pragma unroll
    for (int i = 0; i < HD / 4; ++i) qr[i] = Num<T>::ld(qp + 4 * i);
  }
  float m = -INFINITY, l = 0.f;
  f32x4 acc[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  __syncthreads();
  __syncthreads();
  __syncthreads();
  int b = 0;
  for (int tile = (lo / WAVE) * WAVE; tile <= pos; tile += WAVE, b ^= 1) {
    const float* k_s = lds + b * tile_floats;
    const float* v_s = k_s + WAVE * KS;
    // scores of keys 16 wave .. 16 wave + 15 of the tile; lane (col, kq) gives key col's dimension 4 i + kq
    f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
    const float* ka = k_s + (16 * wave + col) * KS + kq * (HD / 4);
#pragma unroll
    for (int n = 0; n < HD / 16; ++n) {
      const float4 a = *reinterpret_cast<const float4*>(ka + 4 * n);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, qr[4 * n], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, qr[4 * n + 1], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, qr[4 * n + 2], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, qr[4 * n + 3], s, 0, 0, 0);
    }
    // element r: key 16 wave + 4 kq + r of the tile, for this lane's head
    float mx = -INFINITY;
    bool valid[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int c = tile + 16 * wave + 4 * kq + r;
      valid[r] = live && c >= lo && c <= pos;
      s[r] = valid[r] ? s[r] * scale : -INFINITY;
      mx = fmaxf(mx, s[r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    if (kq == 0) mx_s[wave * 16 + col] = mx;
    __syncthreads();
    const float m_new = fmaxf(fmaxf(m, fmaxf(mx_s[col], mx_s[16 + col])), fmaxf(mx_s[32 + col], mx_s[48 + col]));
    const float alpha = live ? expf(m - m_new) : 1.f;       // exp(-inf) = 0 on the first tile
#pragma unroll
    for (int r = 0; r < 4; ++r) p_s[(16 * wave + 4 * kq + r) * 16 + col] = valid[r] ? expf(s[r] - m_new) : 0.f;
    __syncthreads();
    float u[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float* pr = p_s + (4 * kq + r) * 16 + col;
      u[r] = (pr[0] + pr[32 * 16]) + (pr[16 * 16] + pr[48 * 16]);                     // key bits 5, then 4
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) u[r] = u[r] + __shfl_xor(u[r], 32, WAVE);             // key bit 3
#pragma unroll
    for (int r = 0; r < 4; ++r) u[r] = u[r] + __shfl_xor(u[r], 16, WAVE);             // key bit 2
    const float sum = (u[0] + u[2]) + (u[1] + u[3]);                                  // key bits 1 and 0
    l = __builtin_fmaf(l, alpha, sum);
    m = live ? m_new : m;
    // values: lane (col, kq) gives dimension 16 blk + col at key 4 j + kq, and its head's probability of that key
    const float* va = v_s + col * VS + kq * (WAVE / 4);
    const float* pb = p_s + kq * 16 + col;
#pragma unroll
    for (int i = 0; i < BPW; ++i) {
      const int blk = wave + HA_COMPUTE * i;
      if (NBLK % HA_COMPUTE != 0 && blk >= NBLK) break;
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][r] = acc[i][r] * alpha;
#pragma unroll
      for (int n = 0; n < 4; ++n) {
        const float4 v = *reinterpret_cast<const float4*>(va + blk * 16 * VS + 4 * n);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(v.x, pb[4 * (4 * n) * 16], acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(v.y, pb[4 * (4 * n + 1) * 16], acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(v.z, pb[4 * (4 * n + 2) * 16], acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(v.w, pb[4 * (4 * n + 3) * 16], acc[i], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  if (!live) return;
  T* op = out + t * out_stride + (int64_t)h * HD;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < BPW; ++i) {
    const int blk = wave + HA_COMPUTE * i;
    if (NBLK % HA_COMPUTE != 0 && blk >= NBLK) break;
#pragma unroll
    for (int r = 0; r < 4; ++r) Num<T>::st(op + blk * 16 + 4 * kq + r, acc[i][r] * inv);
  }
}

// out: [T, nh*hd] (row stride out_stride elements); q: rows of stride q_stride (the fused q|k|v
// buffer); k_pages: [pages, nkv, page_size, hd]; v_pages: [pages, nkv, hd, page_size]; block_table: [entries, table_width];
// token_entry, positions: [T].  tokens_per_workgroup: how many neighbouring tokens of the step share a workgroup and,
// where they are of one request, its tiles of keys and values (1 for steps of single tokens; 0: the library chooses,
// which for steps of 32 tokens and more means two kernels: the matrix cores for a request's 8 tokens and more, a
// wavefront per token and head for fewer; -1: as 0, and the caller knows that every request of the step has at least 8
// tokens in it, which saves the second kernel); a token's result does not depend on it.  few_tokens_workgroups: a step
// that makes no more workgroups of a token and a kv head than this goes whole to the kernel for single tokens;
// fill_workgroups: the kernel for portions takes as many wavefronts to a workgroup as still leave this many workgroups
// (both decide speed only; the caller's table of thresholds holds them).
extern "C" int ga_paged_attention_generic(void* out, int64_t out_stride, const void* q,
                                          int64_t q_stride, const void* k_pages,
                                          const void* v_pages, const void* block_table,
                                          int table_width, const void* token_entry,
                                          const void* positions, int tokens, int nh, int nkv, int hd,
                                          int page_size, int window, float scale, int is_bf16,
                                          int tokens_per_workgroup, int few_tokens_workgroups,
                                          int fill_workgroups, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hd > MAX_HD || hd <= 0 || nkv <= 0 || nh % nkv != 0 || page_size <= 0) return -1;
  const int group = nh / nkv;
  int min_run = 0;            // > 0: the runs of that many tokens and more have gone to the matrix cores
  // 16-byte loads where a key's dimensions and a page's keys come in whole vectors at 16-byte addresses
  const int vec = is_bf16 ? 8 : 4;
  const bool wide = hd % vec == 0 && page_size % vec == 0 && WAVE % page_size == 0 &&
                    ((uintptr_t)k_pages % 16 == 0) && ((uintptr_t)v_pages % 16 == 0);
  // Steps that hold prompt portions, at the head sizes it is built for: the kernel on the matrix cores.  A workgroup
  // holds tq groups of tokens times hpw heads of a kv group, which share its tiles: as many wavefronts (12, 8, 4, 2,
  // 1) as still leave one and a half workgroups to every compute unit, so that the units that finish the first tokens
  // of a prompt, which see few keys, find more work (measured: that weighs more than the sharing); whole kv groups
  // or divisors of them, so that no wavefront is without a head.
  const bool long_runs_only = tokens_per_workgroup < 0;
  if (long_runs_only) tokens_per_workgroup = 0;
  // A step of few tokens, whatever they are: a workgroup per token and kv head (the heads kernel below) while there
  // are no more than two of them to a compute unit.  Its four wavefronts share a tile's keys, where the kernel for
  // prompt portions has one wavefront walk them; that one wins by the tiles its tokens share once there are many
  // (measured at contexts of 512 and 4,096: 12 heads in 2 groups up to 256 tokens, 28 in 4 up to 128, 16 in 16 up to 32).
  if (tokens_per_workgroup == 0 && wide && hd % 16 == 0 && hd <= 128 && (int64_t)tokens * nkv * ((group + 15) / 16) <= few_tokens_workgroups)
    tokens_per_workgroup = 1;
  if (tokens_per_workgroup == 0 && tokens >= 2 * MA_COLS && hd % 16 == 0 && hd <= 128) {
    int tq = 1, hpw = 1;
    auto workgroups = [&](int tq_, int hpw_) {
      return ((int64_t)(tokens + tq_ * MA_COLS - 1) / (tq_ * MA_COLS)) * nkv * ((group + hpw_ - 1) / hpw_);
    };
    static const int wavefronts[] = {MA_MAX_COMPUTE, 8, 4, 2, 1};
    for (int most : wavefronts) {
      int best = -1;
      for (int h = 1; h <= group && h <= most; ++h) {
        if (group % h != 0) continue;
        const int t = most / h, key = 2 * (t * h + (h == group ? 1 : 0));      // a whole kv group counts for one more
        if (key >= best) best = key, tq = t, hpw = h;                           // among equals, more heads
      }
      if (workgroups(tq, hpw) >= fill_workgroups) break;
    }
    const int head_blocks = (group + hpw - 1) / hpw, waves = tq * hpw;
    const size_t lds = sizeof(float) * (2 * ((size_t)WAVE * (hd + KPAD) + (size_t)hd * VS) + (size_t)waves * (WAVE / 2) * MA_COLS) +
                       sizeof(int64_t) * (2 * WAVE + 1);
    const int64_t workgroup_count = ((int64_t)(tokens + tq * MA_COLS - 1) / (tq * MA_COLS)) * nkv * head_blocks;
    dim3 grid((unsigned)workgroup_count), block(WAVE * (waves + MA_LOADERS));
    bool launched = workgroup_count <= 0x7fffffff;
#define LAUNCH_MATRIX(TT, VV, HH)                                                                                    \
  do {                                                                                                               \
    const void* fn = (const void*)paged_attention_matrix_kernel<TT, VV, HH>;                                         \
    if (lds > 48 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { \
      (void)hipGetLastError();                                                                                       \
      launched = false;                                                                                              \
      break;                                                                                                         \
    }                                                                                                                \
    hipLaunchKernelGGL((paged_attention_matrix_kernel<TT, VV, HH>), grid, block, lds, stream, (TT*)out, out_stride,  \
                       (const TT*)q, q_stride, (const TT*)k_pages, (const TT*)v_pages, (const int32_t*)block_table,  \
                       table_width, (const int32_t*)token_entry, (const int32_t*)positions, tokens, nh, nkv,          \
                       page_size, window, scale, tq, hpw);                                                           \
  } while (0)
#define LAUNCH_MATRIX_HD(TT, VV)                                                                                     \
  do {                                                                                                               \
    switch (hd) {                                                                                                    \
      case 16: LAUNCH_MATRIX(TT, VV, 16); break;                                                                     \
      case 32: LAUNCH_MATRIX(TT, VV, 32); break;                                                                     \
      case 48: LAUNCH_MATRIX(TT, VV, 48); break;                                                                     \
      case 64: LAUNCH_MATRIX(TT, VV, 64); break;                                                                     \
      case 80: LAUNCH_MATRIX(TT, VV, 80); break;                                                                     \
      case 96: LAUNCH_MATRIX(TT, VV, 96); break;                                                                     \
      case 112: LAUNCH_MATRIX(TT, VV, 112); break;                                                                   \
      default: LAUNCH_MATRIX(TT, VV, 128); break;                                                                    \
    }                                                                                                                \
  } while (0)
    if (launched) {
      if (is_bf16) {
        if (wide) LAUNCH_MATRIX_HD(bf16_t, 8);
        else LAUNCH_MATRIX_HD(bf16_t, 1);
      } else {
        if (wide) LAUNCH_MATRIX_HD(float, 4);
        else LAUNCH_MATRIX_HD(float, 1);
      }
    }
#undef LAUNCH_MATRIX_HD
#undef LAUNCH_MATRIX
    if (launched) {
      const int rc = GA_CHECK_LAUNCH();
      if (rc != 0 || long_runs_only) return rc;
      min_run = MA_MIN_RUN;                          // the kernel below takes the shorter runs, a token to a workgroup
      tokens_per_workgroup = 1;
    }
  }
  // Single tokens (a decode step, or the short runs beside the matrix kernel's), 16-byte loads, the same head sizes:
  // the heads of a kv group as the columns of matrix-core products.
  if (tokens_per_workgroup == 1 && wide && hd % 16 == 0 && hd <= 128) {
    const int head_blocks = (group + 15) / 16;
    const size_t lds = sizeof(float) * (2 * ((size_t)WAVE * (hd + KPAD) + (size_t)hd * VS) + (size_t)WAVE * 16 + HA_COMPUTE * 16) +
                       sizeof(int64_t) * (2 * WAVE + 1);
    dim3 grid((unsigned)tokens, nkv * head_blocks), block(WAVE * (HA_COMPUTE + HA_LOADERS));
    bool launched = (int64_t)nkv * head_blocks <= 65535;
#define LAUNCH_HEADS(TT, VV, HH)                                                                                     \
  do {                                                                                                               \
    const void* fn = (const void*)paged_attention_heads_kernel<TT, VV, HH>;                                          \
    if (lds > 48 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { \
      (void)hipGetLastError();                                                                                       \
      launched = false;                                                                                              \
      break;                                                                                                         \
    }                                                                                                                \
    hipLaunchKernelGGL((paged_attention_heads_kernel<TT, VV, HH>), grid, block, lds, stream, (TT*)out, out_stride,   \
                       (const TT*)q, q_stride, (const TT*)k_pages, (const TT*)v_pages, (const int32_t*)block_table,  \
                       table_width, (const int32_t*)token_entry, (const int32_t*)positions, tokens, nh, nkv,          \
                       page_size, window, scale, min_run);                                                           \
  } while (0)
#define LAUNCH_HEADS_HD(TT, VV)                                                                                      \
  do {                                                                                                               \
    switch (hd) {                                                                                                    \
      case 16: LAUNCH_HEADS(TT, VV, 16); break;                                                                      \
      case 32: LAUNCH_HEADS(TT, VV, 32); break;                                                                      \
      case 48: LAUNCH_HEADS(TT, VV, 48); break;                                                                      \
      case 64: LAUNCH_HEADS(TT, VV, 64); break;                                                                      \
      case 80: LAUNCH_HEADS(TT, VV, 80); break;                                                                      \
      case 96: LAUNCH_HEADS(TT, VV, 96); break;                                                                      \
      case 112: LAUNCH_HEADS(TT, VV, 112); break;                                                                    \
      default: LAUNCH_HEADS(TT, VV, 128); break;                                                                     \
    }                                                                                                                \
  } while (0)
    if (launched) {
      if (is_bf16) LAUNCH_HEADS_HD(bf16_t, 8);
      else LAUNCH_HEADS_HD(float, 4);
    }
#undef LAUNCH_HEADS_HD
#undef LAUNCH_HEADS
    if (launched) return GA_CHECK_LAUNCH();         // else: the kernel below
  }
  const int hpw = group < GA_MAX_WAVES ? group : GA_MAX_WAVES, head_blocks = (group + hpw - 1) / hpw;
  int tq = tokens_per_workgroup > 0 ? tokens_per_workgroup : 4;
  if (tq * hpw > GA_MAX_WAVES) tq = GA_MAX_WAVES / hpw;
  if (tq > tokens) tq = tokens;
  const int waves = tq * hpw;
  const size_t tile_bytes = sizeof(float) * ((size_t)WAVE * (hd + KPAD) + (size_t)hd * VS);
  const size_t rest_bytes = sizeof(float) * ((size_t)waves * hd + (size_t)waves * WAVE) + sizeof(int32_t) * 2 * WAVE;
  if ((int64_t)nkv * head_blocks > 65535) return -3;
  // A workgroup with few wavefronts that compute (a decoded token: the heads of one kv group) gets further ones that
  // only help to load: a tile's loads are then all under way at once, and a tile's time is one trip to memory.
  int total_waves = waves;
  const int vectors = WAVE * hd / (wide ? vec : 1);                   // loads of a tile's keys (and as many of its values)
  while (total_waves < GA_MAX_WAVES && total_waves * WAVE * GA_BATCH < vectors) ++total_waves;
  dim3 grid((tokens + tq - 1) / tq, nkv * head_blocks), block(WAVE * total_waves);
  // Few workgroups (a decode step: they cannot fill the chip, and each walks its keys alone): two tile buffers, the
  // next tile loaded while this one is multiplied, where both fit and a thread's one batch of loads is a whole tile.
  // (Beside the matrix kernel the workgroups that find work are those of a few single tokens: the same.)
  const bool pipelined = ((int64_t)grid.x * grid.y <= 256 || min_run > 0) && 2 * tile_bytes + rest_bytes <= 150 * 1024 &&
                         GA_MAX_WAVES - waves >= waves;
  if (pipelined) block.x = WAVE * GA_MAX_WAVES;
  const size_t lds = (pipelined ? 2 : 1) * tile_bytes + rest_bytes;
#define LAUNCH(TT, VV, PP)                                                                                           \
  do {                                                                                                               \
    const void* fn = (const void*)paged_attention_generic_kernel<TT, VV, PP>;                                        \
    if (lds > 48 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
      return -4;                                                                                                     \
    hipLaunchKernelGGL((paged_attention_generic_kernel<TT, VV, PP>), grid, block, lds, stream, (TT*)out, out_stride, \
                       (const TT*)q, q_stride, (const TT*)k_pages, (const TT*)v_pages, (const int32_t*)block_table,  \
                       table_width, (const int32_t*)token_entry, (const int32_t*)positions, tokens, nh, nkv, hd,      \
                       page_size, window, scale, tq, hpw, min_run);                                                  \
  } while (0)
  if (is_bf16) {
    if (wide && pipelined) LAUNCH(bf16_t, 8, true);
    else if (wide) LAUNCH(bf16_t, 8, false);
    else if (pipelined) LAUNCH(bf16_t, 1, true);
    else LAUNCH(bf16_t, 1, false);
  } else {
    if (wide && pipelined) LAUNCH(float, 4, true);
    else if (wide) LAUNCH(float, 4, false);
    else if (pipelined) LAUNCH(float, 1, true);
    else LAUNCH(float, 1, false);
  }
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
