// Paged attention, the general kernel: any mix of prompt portions and single decoded tokens, any
// head size up to 256, full or windowed, 32-bit or bfloat16 storage with
// 32-bit scores, softmax and accumulators.  It is the whole of the 32-bit path and the fallback of
// the bfloat16 path.
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
#include "common.cuh"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations

#define MAX_HD 256

template <typename T>
__global__ void paged_attention_generic_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ token_entry, const int32_t* __restrict__ positions, int nh, int nkv,
    int hd, int page_size, int window, float scale) {
  __shared__ float q_s[MAX_HD];
  __shared__ float p_s[WAVE];
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int g = h / (nh / nkv);
  const int lane = threadIdx.x;
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* bt = block_table + (int64_t)token_entry[t] * table_width;
  const T* qp = q + t * q_stride + (int64_t)h * hd;
  for (int d = lane; d < hd; d += WAVE) q_s[d] = Num<T>::ld(qp + d);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[MAX_HD / WAVE];
#pragma unroll
  for (int i = 0; i < MAX_HD / WAVE; ++i) acc[i] = 0.f;

  for (int tile = (lo / WAVE) * WAVE; tile <= pos; tile += WAVE) {
    const int c = tile + lane;
    const bool valid = c >= lo && c <= pos;
    float s = -INFINITY;
    if (valid) {
      const int64_t page = bt[c / page_size];
      const T* kp = k_pages + ((page * nkv + g) * page_size + (c % page_size)) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot += q_s[d] * Num<T>::ld(kp + d);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));   // finite: every tile holds at least one valid key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);         // exp(-inf) = 0 on the first tile
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    p_s[lane] = p;
    __syncthreads();
    const int j0 = lo > tile ? lo - tile : 0;
    const int j1 = pos - tile < WAVE - 1 ? pos - tile : WAVE - 1;
#pragma unroll
    for (int i = 0; i < MAX_HD / WAVE; ++i) {
      const int d = lane + i * WAVE;
      if (d < hd) {
        float a = acc[i] * alpha;
        for (int j = j0; j <= j1; ++j) {
          const int cc = tile + j;
          const int64_t page = bt[cc / page_size];
          const T* vp = v_pages + ((page * nkv + g) * hd + d) * page_size + (cc % page_size);
          a += p_s[j] * Num<T>::ld(vp);
        }
        acc[i] = a;
      }
    }
  }
  T* op = out + t * out_stride + (int64_t)h * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < MAX_HD / WAVE; ++i) {
    const int d = lane + i * WAVE;
    if (d < hd) Num<T>::st(op + d, acc[i] * inv);
  }
}

// out: [T, nh*hd] (row stride out_stride elements); q: rows of stride q_stride (the fused q|k|v
// buffer); k_pages: [pages, nkv, page_size, hd]; v_pages: [pages, nkv, hd, page_size]; block_table: [entries, table_width];
// token_entry, positions: [T].
extern "C" int ga_paged_attention_generic(void* out, int64_t out_stride, const void* q,
                                          int64_t q_stride, const void* k_pages,
                                          const void* v_pages, const void* block_table,
                                          int table_width, const void* token_entry,
                                          const void* positions, int tokens, int nh, int nkv, int hd,
                                          int page_size, int window, float scale, int is_bf16,
                                          hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hd > MAX_HD || hd <= 0 || nkv <= 0 || nh % nkv != 0) return -1;
  dim3 grid(tokens, nh), block(WAVE);
  if (is_bf16)
    hipLaunchKernelGGL(paged_attention_generic_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out,
                       out_stride, (const bf16_t*)q, q_stride, (const bf16_t*)k_pages,
                       (const bf16_t*)v_pages, (const int32_t*)block_table, table_width,
                       (const int32_t*)token_entry, (const int32_t*)positions, nh, nkv, hd,
                       page_size, window, scale);
  else
    hipLaunchKernelGGL(paged_attention_generic_kernel<float>, grid, block, 0, stream, (float*)out,
                       out_stride, (const float*)q, q_stride, (const float*)k_pages,
                       (const float*)v_pages, (const int32_t*)block_table, table_width,
                       (const int32_t*)token_entry, (const int32_t*)positions, nh, nkv, hd,
                       page_size, window, scale);
  return GA_CHECK_LAUNCH();
}
