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
#include "common.cuh"

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

// The same with 16-byte accesses: one workgroup per token walks all heads; an item is a chunk of V
// consecutive pairs (j, j + half) of a q or k head, a chunk of the unrotated tail, or a chunk of a v head.
// For rotary_dim / 2, head_dim - rotary_dim and head_dim multiples of V = 16 / sizeof(T).
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_vec_kernel(
    T* __restrict__ qkv, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int64_t* __restrict__ slot_mapping, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int nh, int nkv, int hd, int rotary_dim, int page_size, int write_kv) {
  constexpr int V = 16 / sizeof(T);
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
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const float l = Num<T>::ld(&lo.e[i]), h = Num<T>::ld(&hi.e[i]);
          const float cj = c[j + i], sj = s[j + i];
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
    } else if (page >= 0) {
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
    if (is_bf16)
      hipLaunchKernelGGL(rope_kv_write_vec_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, (bf16_t*)qkv,
                         (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,
                         (const int64_t*)slot_mapping, (bf16_t*)k_pages, (bf16_t*)v_pages, nh, nkv, hd, rotary_dim,
                         page_size, write_kv);
    else
      hipLaunchKernelGGL(rope_kv_write_vec_kernel<float>, dim3(tokens), dim3(256), 0, stream, (float*)qkv,
                         (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,
                         (const int64_t*)slot_mapping, (float*)k_pages, (float*)v_pages, nh, nkv, hd, rotary_dim,
                         page_size, write_kv);
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
