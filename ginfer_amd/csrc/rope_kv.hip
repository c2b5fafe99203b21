// Rotary position encoding (NeoX pairing) of q and k, and the write of k and v into the paged
// cache, in one launch over the fused q|k|v projection.
//   o[j]      = x[j] * cos[p, j] - x[j + half] * sin[p, j]
//   o[j+half] = x[j] * sin[p, j] + x[j + half] * cos[p, j]          j < half = rotary_dim / 2
// with p = positions[t]; elements past rotary_dim pass through.  32-bit arithmetic on 32-bit
// tables, one rounding.  Formula: ginfer/core/op/kernels/cuda/rope_kernel.cu:83-102; cache write:
// ginfer/core/op/kernels/cuda/store_kvcache_kernel.cu:19-30 (which indexes with 32-bit ints; the
// offsets here are 64-bit).
// Cache layout of one layer: keys  k_pages[page][kv_head][slot_in_page][head_dim],
//                            values v_pages[page][kv_head][head_dim][slot_in_page]  (transposed, so
// that the matrix-core attention kernels read 8 consecutive keys of one dimension in one 16-byte
// load).  The slot of token t is slot_mapping[t] = page * page_size + slot_in_page, or -1 to write
// nothing for that token.
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                                     const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                     const int64_t* __restrict__ slot_mapping,
                                     T* __restrict__ k_pages, T* __restrict__ v_pages, int nh,
                                     int nkv, int hd, int rotary_dim, int page_size, int write_kv) {
  const int64_t t = blockIdx.x;
  const int head = blockIdx.y;  // 0..nh-1: q; nh..nh+nkv-1: k; then v
  const int half = rotary_dim >> 1;
  T* x = qkv + (t * (nh + 2 * nkv) + head) * (int64_t)hd;
  const int p = positions[t];
  const bool is_q = head < nh, is_k = !is_q && head < nh + nkv;
  T* dst = nullptr;   // k: the slot's row of head_dim; v: the slot's column, elements page_size apart
  if (!is_q && write_kv) {
    const int64_t slot = slot_mapping[t];
    if (slot >= 0) {
      const int g = is_k ? head - nh : head - nh - nkv;
      int64_t page, off;
      slot_page(slot, page_size, page, off);
      dst = is_k ? k_pages + ((page * nkv + g) * page_size + off) * hd
                 : v_pages + (page * nkv + g) * (int64_t)hd * page_size + off;
    }
  }
  if (is_q || is_k) {
    const float* c = cos_t + (int64_t)p * half;
    const float* s = sin_t + (int64_t)p * half;
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
      const float lo = Num<T>::ld(x + j), hi = Num<T>::ld(x + j + half);
      const float cj = c[j], sj = s[j];
      const float olo = lo * cj - hi * sj, ohi = lo * sj + hi * cj;
      Num<T>::st(x + j, olo);
      Num<T>::st(x + j + half, ohi);
      if (dst) {
        Num<T>::st(dst + j, olo);
        Num<T>::st(dst + j + half, ohi);
      }
    }
    if (dst)
      for (int j = rotary_dim + threadIdx.x; j < hd; j += blockDim.x) dst[j] = x[j];
  } else if (dst) {
    for (int j = threadIdx.x; j < hd; j += blockDim.x) dst[(int64_t)j * page_size] = x[j];
  }
}

// The values of ROPE_ROWS consecutive tokens of the step, written by one workgroup.  In the transposed pages an
// element of v lies page_size elements from the next of its token, so a token alone writes 2 or 4 bytes at a time,
// each into a 32-byte sector of its own.  Here the tokens' v rows wait in LDS, and the thread that owns one
// (kv head, dim) writes the tokens whose slots follow each other inside a page in one store of up to 16 bytes: the
// tokens of a prompt portion do.  Which tokens form a run depends on the slots alone, so the threads branch together.
// Dynamic LDS: ROPE_ROWS * nkv * hd elements.
#define ROPE_ROWS 8
#define ROPE_VALUE_BLOCKS_FROM 512
template <typename T>
__device__ __forceinline__ void write_values_in_runs(const T* __restrict__ qkv, const int64_t* __restrict__ slot_mapping,
                                                     T* __restrict__ v_pages, int tokens, int64_t t0, int nh, int nkv,
                                                     int hd, int page_size) {
  constexpr int V = 16 / sizeof(T);
  extern __shared__ __attribute__((aligned(16))) unsigned char rows_lds[];
  T* v_rows = reinterpret_cast<T*>(rows_lds);                       // [ROPE_ROWS][nkv * hd]
  __shared__ int64_t s_slot[ROPE_ROWS];
  const int rows = tokens - t0 < ROPE_ROWS ? (int)(tokens - t0) : ROPE_ROWS;
  const int width = nkv * hd, chunks = width / V;
  if ((int)threadIdx.x < rows) s_slot[threadIdx.x] = slot_mapping[t0 + threadIdx.x];
  for (int idx = threadIdx.x; idx < rows * chunks; idx += blockDim.x) {
    const int r = idx / chunks, ch = idx % chunks;
    *reinterpret_cast<uint4*>(v_rows + r * width + ch * V) =
        *reinterpret_cast<const uint4*>(qkv + (t0 + r) * (int64_t)(nh + 2 * nkv) * hd + (int64_t)(nh + nkv) * hd + ch * V);
  }
  __syncthreads();
  for (int pair = threadIdx.x; pair < width; pair += blockDim.x) {
    const int g = pair / hd, j = pair % hd;
    const T* mine = v_rows + pair;                                  // this (kv head, dim) of row r: mine[r * width]
    int r = 0;
    while (r < rows) {                                              // the same walk in every thread
      const int64_t slot = s_slot[r];
      if (slot < 0) {
        ++r;
        continue;
      }
      int64_t page, off;
      slot_page(slot, page_size, page, off);
      int len = 1;                                                  // tokens of the run: a power of two, at most V
      for (int c = V; c > 1; c >>= 1) {
        if (r + c > rows || page_size % c || off % c) continue;
        bool follow = true;
        for (int i = 1; i < c; ++i) follow = follow && s_slot[r + i] == slot + i;
        if (follow) {
          len = c;
          break;
        }
      }
      T* dst = v_pages + ((page * nkv + g) * (int64_t)hd + j) * page_size + off;
      union { uint4 u; uint2 d; uint32_t w; T e[V]; } out;
      if (len == V) {
#pragma unroll
        for (int i = 0; i < V; ++i) out.e[i] = mine[(r + i) * width];
        *reinterpret_cast<uint4*>(dst) = out.u;
      } else if (len * sizeof(T) == 8) {
#pragma unroll
        for (int i = 0; i < (int)(8 / sizeof(T)); ++i) out.e[i] = mine[(r + i) * width];
        *reinterpret_cast<uint2*>(dst) = out.d;
      } else if (len == 2 && sizeof(T) == 2) {
#pragma unroll
        for (int i = 0; i < 2; ++i) out.e[i] = mine[(r + i) * width];
        *reinterpret_cast<uint32_t*>(dst) = out.w;
      } else {
        len = 1;
        dst[0] = mine[r * width];
      }
      r += len;
    }
  }
}

// The same with 16-byte accesses: one workgroup per token walks all heads; an item is a chunk of V
// consecutive pairs (j, j + half) of a q or k head, a chunk of the unrotated tail, or a chunk of a v head.
// For rotary_dim / 2, head_dim - rotary_dim and head_dim multiples of V = 16 / sizeof(T).
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_vec_kernel(
    T* __restrict__ qkv, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int64_t* __restrict__ slot_mapping, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int nh, int nkv, int hd, int rotary_dim, int page_size, int write_kv, int tokens,
    int value_blocks) {
  constexpr int V = 16 / sizeof(T);
  if (value_blocks && (int)blockIdx.x >= tokens) {
    write_values_in_runs<T>(qkv, slot_mapping, v_pages, tokens, ((int64_t)blockIdx.x - tokens) * ROPE_ROWS, nh, nkv, hd,
                            page_size);
    return;
  }
  const int64_t t = blockIdx.x;
  const int half = rotary_dim >> 1;
  const int rot_chunks = half / V, tail_chunks = (hd - rotary_dim) / V, v_chunks = hd / V;
  const int per_head = rot_chunks + tail_chunks;
  const int qk_items = (nh + nkv) * per_head;
  const int total = qk_items + nkv * v_chunks;
  const int p = positions[t];
  const float* c = cos_t + (int64_t)p * half;
  const float* s = sin_t + (int64_t)p * half;
  T* row = qkv + t * (int64_t)(nh + 2 * nkv) * hd;
  int64_t page = -1, off = 0;
  if (write_kv) {
    const int64_t slot = slot_mapping[t];
    if (slot >= 0) {
      slot_page(slot, page_size, page, off);
    }
  }
  for (int item = threadIdx.x; item < total; item += blockDim.x) {
    if (item < qk_items) {
      const int head = item / per_head, ch = item % per_head;
      T* x = row + (int64_t)head * hd;
      T* dst = (head >= nh && page >= 0) ? k_pages + ((page * nkv + (head - nh)) * page_size + off) * hd : nullptr;
      if (ch < rot_chunks) {
        const int j = ch * V;
        union { uint4 u; T e[V]; } lo, hi, olo, ohi;
        lo.u = *reinterpret_cast<const uint4*>(x + j);
        hi.u = *reinterpret_cast<const uint4*>(x + j + half);
        // the tables' rows in 16-byte loads too (a row starts at a multiple of V floats, and so does j)
        union { float4 q[V / 4]; float e[V]; } cv, sv;
#pragma unroll
        for (int i = 0; i < V / 4; ++i) {
          cv.q[i] = *reinterpret_cast<const float4*>(c + j + 4 * i);
          sv.q[i] = *reinterpret_cast<const float4*>(s + j + 4 * i);
        }
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const float l = Num<T>::ld(&lo.e[i]), h = Num<T>::ld(&hi.e[i]);
          const float cj = cv.e[i], sj = sv.e[i];
          Num<T>::st(&olo.e[i], l * cj - h * sj);
          Num<T>::st(&ohi.e[i], l * sj + h * cj);
        }
        *reinterpret_cast<uint4*>(x + j) = olo.u;
        *reinterpret_cast<uint4*>(x + j + half) = ohi.u;
        if (dst) {
          *reinterpret_cast<uint4*>(dst + j) = olo.u;
          *reinterpret_cast<uint4*>(dst + j + half) = ohi.u;
        }
      } else if (dst) {
        const int j = rotary_dim + (ch - rot_chunks) * V;
        *reinterpret_cast<uint4*>(dst + j) = *reinterpret_cast<const uint4*>(x + j);
      }
    } else if (page >= 0 && !value_blocks) {
      const int vi = item - qk_items;
      const int g = vi / v_chunks, j = (vi % v_chunks) * V;
      union { uint4 u; T e[V]; } val;
      val.u = *reinterpret_cast<const uint4*>(row + (int64_t)(nh + nkv + g) * hd + j);
      T* dst = v_pages + ((page * nkv + g) * (int64_t)hd + j) * page_size + off;
#pragma unroll
      for (int i = 0; i < V; ++i) dst[(int64_t)i * page_size] = val.e[i];
    }
  }
}

extern "C" int ga_rope_kv_write(void* qkv, const void* positions, const void* cos_t,
                                const void* sin_t, const void* slot_mapping, void* k_pages,
                                void* v_pages, int tokens, int nh, int nkv, int hd, int rotary_dim,
                                int page_size, int write_kv, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  const int v = is_bf16 ? 8 : 4;
  if ((rotary_dim / 2) % v == 0 && (hd - rotary_dim) % v == 0 && hd % v == 0) {
    // Further workgroups that write the values of ROPE_ROWS tokens each, where their rows fit in LDS and the step is
    // long (measured on MI355X, 12 + 2 x 2 heads of 128, slots 5 past a page's start: 8.2 -> 7.7 us at 2,048 tokens,
    // 37 -> 31 at 16,384; at 256 tokens, where the launch is what counts, 3.6 -> 4.2)
    const size_t rows_lds = (size_t)ROPE_ROWS * nkv * hd * (is_bf16 ? 2 : 4);
    const int value_blocks =
        (write_kv && tokens >= ROPE_VALUE_BLOCKS_FROM && rows_lds <= 32 * 1024) ? (tokens + ROPE_ROWS - 1) / ROPE_ROWS : 0;
    dim3 grid(tokens + value_blocks), block(256);
    if (is_bf16)
      hipLaunchKernelGGL(rope_kv_write_vec_kernel<bf16_t>, grid, block, value_blocks ? rows_lds : 0, stream,
                         (bf16_t*)qkv, (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,
                         (const int64_t*)slot_mapping, (bf16_t*)k_pages, (bf16_t*)v_pages, nh, nkv, hd, rotary_dim,
                         page_size, write_kv, tokens, value_blocks);
    else
      hipLaunchKernelGGL(rope_kv_write_vec_kernel<float>, grid, block, value_blocks ? rows_lds : 0, stream,
                         (float*)qkv, (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,
                         (const int64_t*)slot_mapping, (float*)k_pages, (float*)v_pages, nh, nkv, hd, rotary_dim,
                         page_size, write_kv, tokens, value_blocks);
    return GA_CHECK_LAUNCH();
  }
  dim3 grid(tokens, nh + 2 * nkv), block(64);
  if (is_bf16)
    hipLaunchKernelGGL(rope_kv_write_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)qkv,
                       (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,
                       (const int64_t*)slot_mapping, (bf16_t*)k_pages, (bf16_t*)v_pages, nh, nkv,
                       hd, rotary_dim, page_size, write_kv);
  else
    hipLaunchKernelGGL(rope_kv_write_kernel<float>, grid, block, 0, stream, (float*)qkv,
                       (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,
                       (const int64_t*)slot_mapping, (float*)k_pages, (float*)v_pages, nh, nkv, hd,
                       rotary_dim, page_size, write_kv);
  return GA_CHECK_LAUNCH();
}

// The same epilogue on a projection that arrives as 32-bit partial sums of a product whose K was split over workgroups
// (parts [n_parts][tokens][(nh + 2 nkv) hd]): the parts are added in ascending order, the bias in 32-bit, q and k are
// rotated on the 32-bit sums (one rounding fewer than rotating the rounded projection), q goes to q_out
// [tokens][nh hd] in bfloat16, k and v straight into the pages.  A workgroup takes one token and one of
// FROM_PARTS_CHUNKS shares of its items (an item: 4 consecutive pairs (j, j + half) of a q or k head, 4 elements of an
// unrotated tail, or 4 elements of a v head), so that few tokens still make workgroups enough.
#define FROM_PARTS_CHUNKS 2
#define FROM_PARTS_MOST 8            // parts at most: their loads are all asked for before the first is added
__global__ __launch_bounds__(256) void rope_kv_from_parts_kernel(
    bf16_t* __restrict__ q_out, const float* __restrict__ parts, int n_parts, const bf16_t* __restrict__ bias,
    const int32_t* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int64_t* __restrict__ slot_mapping, bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, int nh, int nkv,
    int hd, int rotary_dim, int page_size, int write_kv, int tokens) {
  constexpr int V = 4;
  const int64_t t = blockIdx.x;
  const int half = rotary_dim >> 1;
  const int rot_chunks = half / V, tail_chunks = (hd - rotary_dim) / V, v_chunks = hd / V;
  const int per_head = rot_chunks + tail_chunks;
  const int qk_items = (nh + nkv) * per_head;
  const int total = qk_items + nkv * v_chunks;
  const int width = (nh + 2 * nkv) * hd;
  const int p = positions[t];
  const float* c = cos_t + (int64_t)p * half;
  const float* s = sin_t + (int64_t)p * half;
  const int64_t part_stride = (int64_t)tokens * width;
  const float* row = parts + t * (int64_t)width;
  int64_t page = -1, off = 0;
  if (write_kv) {
    const int64_t slot = slot_mapping[t];
    if (slot >= 0) slot_page(slot, page_size, page, off);
  }
  // the parts' four values of column `at`, all asked for at once (n_parts is the same for every lane)
  auto ask = [&](float4 (&v)[FROM_PARTS_MOST], int at) {
#pragma unroll
    for (int q = 0; q < FROM_PARTS_MOST; ++q)
      if (q < n_parts) v[q] = *reinterpret_cast<const float4*>(row + q * part_stride + at);
  };
  // ... added in ascending order, then the bias
  auto add_up = [&](float (&x)[V], const float4 (&v)[FROM_PARTS_MOST], int at) {
    x[0] = x[1] = x[2] = x[3] = 0.f;
#pragma unroll
    for (int q = 0; q < FROM_PARTS_MOST; ++q)
      if (q < n_parts) {
        x[0] += v[q].x; x[1] += v[q].y; x[2] += v[q].z; x[3] += v[q].w;
      }
    if (bias) {
      union { uint2 u; bf16_t e[V]; } bv;
      bv.u = *reinterpret_cast<const uint2*>(bias + at);
#pragma unroll
      for (int i = 0; i < V; ++i) x[i] += bf16_to_f32(bv.e[i]);
    }
  };
  for (int item = blockIdx.y * blockDim.x + threadIdx.x; item < total; item += gridDim.y * blockDim.x) {
    if (item < qk_items) {
      const int head = item / per_head, ch = item % per_head;
      bf16_t* dst = head < nh ? q_out + t * (int64_t)nh * hd + (int64_t)head * hd
                              : (page >= 0 ? k_pages + ((page * nkv + (head - nh)) * page_size + off) * hd : nullptr);
      if (!dst) continue;
      if (ch < rot_chunks) {
        const int j = ch * V;
        float4 plo[FROM_PARTS_MOST], phi[FROM_PARTS_MOST];
        ask(plo, head * hd + j);
        ask(phi, head * hd + j + half);
        const float4 cv = *reinterpret_cast<const float4*>(c + j), sv = *reinterpret_cast<const float4*>(s + j);
        float lo[V], hi[V];
        add_up(lo, plo, head * hd + j);
        add_up(hi, phi, head * hd + j + half);
        const float ce[V] = {cv.x, cv.y, cv.z, cv.w}, se[V] = {sv.x, sv.y, sv.z, sv.w};
        union { uint2 u; bf16_t e[V]; } olo, ohi;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          olo.e[i] = f32_to_bf16(lo[i] * ce[i] - hi[i] * se[i]);
          ohi.e[i] = f32_to_bf16(lo[i] * se[i] + hi[i] * ce[i]);
        }
        *reinterpret_cast<uint2*>(dst + j) = olo.u;
        *reinterpret_cast<uint2*>(dst + j + half) = ohi.u;
      } else {
        const int j = rotary_dim + (ch - rot_chunks) * V;
        float4 px[FROM_PARTS_MOST];
        ask(px, head * hd + j);
        float x[V];
        add_up(x, px, head * hd + j);
        union { uint2 u; bf16_t e[V]; } o;
#pragma unroll
        for (int i = 0; i < V; ++i) o.e[i] = f32_to_bf16(x[i]);
        *reinterpret_cast<uint2*>(dst + j) = o.u;
      }
    } else if (page >= 0) {
      const int vi = item - qk_items;
      const int g = vi / v_chunks, j = (vi % v_chunks) * V;
      float4 px[FROM_PARTS_MOST];
      ask(px, (nh + nkv + g) * hd + j);
      float x[V];
      add_up(x, px, (nh + nkv + g) * hd + j);
      bf16_t* dst = v_pages + ((page * nkv + g) * (int64_t)hd + j) * page_size + off;
#pragma unroll
      for (int i = 0; i < V; ++i) dst[(int64_t)i * page_size] = f32_to_bf16(x[i]);
    }
  }
}

// parts float [n_parts][tokens][(nh + 2 nkv) hd]; bias bfloat16 [(nh + 2 nkv) hd] or null; q_out bfloat16 [tokens][nh hd];
// the rest as ga_rope_kv_write.  rotary_dim / 2, head_dim - rotary_dim and head_dim multiples of 4; at most 8 parts.
extern "C" int ga_rope_kv_from_parts(void* q_out, const void* parts, int n_parts, const void* bias,
                                     const void* positions, const void* cos_t, const void* sin_t,
                                     const void* slot_mapping, void* k_pages, void* v_pages, int tokens, int nh, int nkv,
                                     int hd, int rotary_dim, int page_size, int write_kv, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (n_parts < 1 || n_parts > FROM_PARTS_MOST || nh <= 0 || nkv <= 0) return -1;
  if ((rotary_dim / 2) % 4 || (hd - rotary_dim) % 4 || hd % 4 || rotary_dim <= 0 || rotary_dim > hd) return -2;
  dim3 grid(tokens, FROM_PARTS_CHUNKS), block(256);
  hipLaunchKernelGGL(rope_kv_from_parts_kernel, grid, block, 0, stream, (bf16_t*)q_out, (const float*)parts, n_parts,
                     (const bf16_t*)bias, (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,
                     (const int64_t*)slot_mapping, (bf16_t*)k_pages, (bf16_t*)v_pages, nh, nkv, hd, rotary_dim, page_size,
                     write_kv, tokens);
  return GA_CHECK_LAUNCH();
}
