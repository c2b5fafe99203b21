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
      const int64_t page = slot / page_size, off = slot - page * page_size;
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

extern "C" int ga_rope_kv_write(void* qkv, const void* positions, const void* cos_t,
                                const void* sin_t, const void* slot_mapping, void* k_pages,
                                void* v_pages, int tokens, int nh, int nkv, int hd, int rotary_dim,
                                int page_size, int write_kv, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
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
