// Entry points of the kernel libraries of ginfer_amd (gfx950), for callers outside Python.
//
// Every source under this folder is built into a shared library of its own (lib<source>.so; the matrix-core
// attention once per head size, libattention_mfma_HEAD_DIM<n>.so).  All entry points are `extern "C"`, take raw
// device pointers and the stream to launch on, check what can be checked on the host, and return 0 or a
// negative number without launching anything.  Sizes are in elements unless bytes are named.  bfloat16 values
// are raw 16-bit patterns.  Nothing here allocates device memory: scratch memory is the caller's (or, for
// ga_sample_rows_static, a static array of the library).
//
// Every source includes this header, so the compiler checks each definition against its declaration.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// ---- embedding.hip: out float [tokens, hidden] = table[ids] (table bfloat16 or float, ids int32)
int ga_embedding_gather(void* out, const void* table, const void* ids, int tokens, int hidden, int is_bf16,
                        hipStream_t stream);

// ---- norm.hip: residual float [num_tokens, hidden] += delta (null, [num_tokens, hidden], or float partial sums
// [delta_parts, num_tokens, hidden] added in order); out = rmsnorm(residual) * gain for all rows, or for the
// int32 `rows` alone (then the residual is left as it is)
int ga_add_rmsnorm(void* out, void* residual, const void* delta, int delta_parts, int num_tokens, const void* gain,
                   const void* rows, int num_rows, int hidden, float eps, int is_bf16, int gain_is_f32,
                   hipStream_t stream);

// ---- rope_kv.hip: NeoX rotation of q and k inside the fused projection [tokens, (nh + 2 nkv) hd], k and v
// written to the pages (keys [page][kv head][slot][dim], values [page][kv head][dim][slot]); slot_mapping int64,
// -1: no write
int ga_rope_kv_write(void* qkv, const void* positions, const void* cos_t, const void* sin_t, const void* slot_mapping,
                     void* k_pages, void* v_pages, int tokens, int nh, int nkv, int hd, int rotary_dim, int page_size,
                     int write_kv, int is_bf16, hipStream_t stream);
// the same on 32-bit partial sums of the projection, parts [n_parts][tokens][(nh + 2 nkv) hd] added in order, then the bias
// (bfloat16 or null): q to q_out [tokens][nh hd] in bfloat16, k and v into the pages
int ga_rope_kv_from_parts(void* q_out, const void* parts, int n_parts, const void* bias, const void* positions,
                          const void* cos_t, const void* sin_t, const void* slot_mapping, void* k_pages, void* v_pages,
                          int tokens, int nh, int nkv, int hd, int rotary_dim, int page_size, int write_kv,
                          hipStream_t stream);

// ---- gemm.hip: C [M, N] = A [M, K] . W [N, K]^T + bias in true 32-bit: the matrix cores' 32-bit instructions (and plain FMA
// for 33 to 64 rows of very wide products), every element one accumulator over ascending k: the same bits whichever
// kernel runs (the 32-bit path; also bfloat16 in)
int ga_gemm_nt(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias, int M, int N, int K,
               int in_bf16, int out_bf16, hipStream_t stream);

// ---- gemm_skinny.hip: bfloat16 products for at most 64 rows on the matrix cores
// What ga_gemm_skinny and ga_qkv_rope_skinny take beside the product itself: a norm folded into the products
// around it.  All null or zero for a plain product.
struct GaSkinnyNorm {
  const float* in_sumsq;   // [M][in_parts]: the rows of A are (h * gain) of a norm whose sums of squares these are
  int in_parts;
  float inv_width, eps;
  float* residual;         // [M][N], row stride ldr: the product is added to it (C is not written)
  int64_t ldr;
  const void* gain;        // [N] of the norm that follows
  int gain_f32;
  void* scaled;            // bfloat16 [M][N], row stride lds
  int64_t lds;
  float* out_sumsq;        // [M][ga_skinny_norm_parts(M, N)]
};
int ga_skinny_norm_parts(int M, int N);
int ga_gemm_skinny(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias, int M, int N, int K,
                   int out_f32, int nt, int ks, int grid_splits, int gated, int pack, const struct GaSkinnyNorm* norm,
                   hipStream_t stream);
int ga_qkv_rope_skinny(void* q_out, const void* A, int64_t lda, const void* W, const void* bias, const void* positions,
                       const void* cos_t, const void* sin_t, const void* slot_mapping, void* k_pages, void* v_pages,
                       int M, int K, int nh, int nkv, int hd, int page_size, int write_kv, int pack,
                       const struct GaSkinnyNorm* norm, hipStream_t stream);

// ---- activation.hip: out [tokens, inter] = silu(gu[:, :inter]) * gu[:, inter:]
int ga_silu_mul(void* out, const void* gu, int tokens, int inter, int is_bf16, hipStream_t stream);
// the same on a product that lies transposed, gu_t [2 inter, tokens] bfloat16; tokens and inter multiples of 8
int ga_silu_mul_transposed(void* out, const void* gu_t, int tokens, int inter, hipStream_t stream);

// ---- attention_generic.hip: every token attends to its request's pages; any head size up to 256, window or 0;
// tokens_per_workgroup neighbouring tokens share a workgroup's tiles of keys and values (0: the library chooses; -1: the
// same, and every request of the step has at least 8 tokens in it); few_tokens_workgroups, fill_workgroups: the two
// thresholds by which the launcher chooses among its kernels (speed only)
int ga_paged_attention_generic(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                               const void* v_pages, const void* block_table, int table_width, const void* token_entry,
                               const void* positions, int tokens, int nh, int nkv, int hd, int page_size, int window,
                               float scale, int is_bf16, int tokens_per_workgroup, int few_tokens_workgroups,
                               int fill_workgroups, hipStream_t stream);

// ---- attention_mfma.hip (one library per head size): bfloat16 on the matrix cores
int ga_attn_head_dim();
int ga_attn_prefill_max_tile_rows();
// single new tokens; workspace_o: n_tokens * nh * num_splits * head_dim floats, workspace_ml: n_tokens * nh *
// num_splits * 2 floats
int ga_attn_decode(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                   const void* v_pages, const void* block_table, int table_width, const void* decode_info, int n_tokens,
                   int nh, int nkv, int page_size, int window, float scale, int split_keys, int num_splits,
                   void* workspace_o, void* workspace_ml, hipStream_t stream);
// rows of prompt portions, in tiles of int32 x 4 = (entry, first row of the step, rows, first position).  parts (or
// null): per tile int32 x 4 = (first key, end of keys, index of the tile's first row among the rows that come in parts,
// part + (number of parts << 16)): the keys of such a tile are dealt to several workgroups, whose partial results
// (part_o: n_part_rows * nh * num_parts * head_dim floats, part_ml: ... * 2) a second kernel merges; part_rows: int32 x 4
// per row in parts, its row of the step first
int ga_attn_prefill(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                    const void* v_pages, const void* block_table, int table_width, const void* tiles, int n_tiles,
                    int tile_rows, int nh, int nkv, int page_size, int window, float scale, int fill_workgroups,
                    int prefer_workgroups, const void* parts, const void* part_rows, int n_part_rows, int num_parts, void* part_o,
                    void* part_ml, hipStream_t stream);

// ---- random_fill.hip: out[i] = mean + std * normal(key, i) for n elements, float or bfloat16: the counter-based
// generator of random_normal.h, which gives the host library (host/random_fill_host.cpp) the same bits
int ga_random_normal_fill(void* out, int64_t n, uint64_t key, float mean, float std, int is_bf16, hipStream_t stream);

// ---- sampling.hip: out int32 [rows]: argmax (lowest index among equals) where temperature is null or 0, else one
// draw from softmax(logits / temperature) by the given uniform number; scratch: ga_sample_scratch_floats floats
int64_t ga_sample_scratch_floats(int rows, int vocab);
int ga_sample_rows(void* out, const void* logits, int64_t row_stride, int rows, int vocab, const void* temperature,
                   const void* uniform, void* scratch, hipStream_t stream);

// ---- sampling.hip, for callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid allocation).  This entry point has no counterpart in the reference, whose argmax takes
// its buffers from the caller's allocator.  ga_sample_rows_static is ga_sample_rows with its scratch in a static
// device array of 196,608 bytes that each GPU holds until the process ends: at most
// ga_sample_rows_static_max_rows() (256) rows a call, more are refused with -2 and nothing is launched
// (ga_sample_rows_static_error(code) says what a negative code means).  It allocates nothing and calls nothing that
// does.  Calls on one GPU share the array: calls that overlap there (other streams, other threads) race.
// ga_sample_rows_static_init() looks the array up on the current device ahead of the first call (optional).
int ga_sample_rows_static_max_rows();
int ga_sample_rows_static_init();
const char* ga_sample_rows_static_error(int code);
int ga_sample_rows_static(void* out, const void* logits, int64_t row_stride, int rows, int vocab,
                          const void* temperature, const void* uniform, hipStream_t stream);

#ifdef __cplusplus
}
#endif
