// Choosing the next token from 32-bit logits, one workgroup per row.
//   temperature == 0: argmax, the lowest index among equal maxima (the reference's reduction,
//     ginfer/core/op/kernels/cuda/argmax_kernel.cu:52-98, keeps whichever equal value its tree meets
//     first; ginfer/model/model.cc:219-220 is where it is used).
//   temperature  > 0: p = softmax(logits / temperature) in 32-bit, and the first index whose running
//     sum of exp((x - max) / temperature) exceeds uniform * total: an inverse-CDF draw from a uniform
//     number the caller supplies, so the choice is a pure function of (logits, temperature, uniform).
// The reference samples greedily only (ginfer/engine/sampling_params.h:5-8).
#include "common.cuh"

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / WAVE)

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(
    int32_t* __restrict__ out, const float* __restrict__ logits, int64_t row_stride, int vocab,
    const float* __restrict__ temperature, const float* __restrict__ uniform) {
  __shared__ float part_f[SAMPLE_WAVES];
  __shared__ int part_i[SAMPLE_WAVES];
  __shared__ float seg_sum[SAMPLE_WAVES];
  __shared__ float walk[2];
  __shared__ int owner_s;
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const float* x = logits + (int64_t)r * row_stride;

  // ---- max and its lowest index: strided (coalesced) reads; a thread meets its indices in ascending order
  // four independent candidates per thread, so that four loads are in flight; merged lowest index first
  float bests[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
  int bests_i[4] = {0x7fffffff, 0x7fffffff, 0x7fffffff, 0x7fffffff};
  for (int i0 = tid; i0 < vocab; i0 += 4 * SAMPLE_THREADS) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * SAMPLE_THREADS;
      v[u] = i < vocab ? x[i] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * SAMPLE_THREADS;
      if (i < vocab && (bests_i[u] == 0x7fffffff || v[u] > bests[u])) { bests[u] = v[u]; bests_i[u] = i; }
    }
  }
  float best = bests[0];
  int best_i = bests_i[0];
#pragma unroll
  for (int u = 1; u < 4; ++u)
    if (bests_i[u] != 0x7fffffff && (best_i == 0x7fffffff || bests[u] > best || (bests[u] == best && bests_i[u] < best_i))) {
      best = bests[u];
      best_i = bests_i[u];
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float b = __shfl_xor(best, o, WAVE);
    const int bi = __shfl_xor(best_i, o, WAVE);
    if (bi != 0x7fffffff && (best_i == 0x7fffffff || b > best || (b == best && bi < best_i))) { best = b; best_i = bi; }
  }
  if (lane == 0) { part_f[wave] = best; part_i[wave] = best_i; }
  __syncthreads();
  float mx = part_f[0];
  int arg = part_i[0];
#pragma unroll
  for (int w = 1; w < SAMPLE_WAVES; ++w) {
    const float b = part_f[w];
    const int bi = part_i[w];
    if (bi != 0x7fffffff && (arg == 0x7fffffff || b > mx || (b == mx && bi < arg))) { mx = b; arg = bi; }
  }
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = arg;
    return;
  }
  // ---- mass of each wavefront's contiguous segment of the vocabulary
  const float inv_t = 1.0f / temp;
  const int seg = ((vocab + SAMPLE_WAVES - 1) / SAMPLE_WAVES + WAVE - 1) / WAVE * WAVE;
  const int sb = wave * seg < vocab ? wave * seg : vocab;
  const int se = sb + seg < vocab ? sb + seg : vocab;
  float sum = 0.f;
  for (int i = sb + lane; i < se; i += WAVE) sum += __expf((x[i] - mx) * inv_t);
  sum = wave_sum(sum);
  if (lane == 0) seg_sum[wave] = sum;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int w = 0; w < SAMPLE_WAVES; ++w) total += seg_sum[w];
    const float target = uniform[r] * total;
    float run = 0.f;
    int owner = SAMPLE_WAVES - 1;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
      if (run + seg_sum[w] > target) { owner = w; break; }
      if (w < SAMPLE_WAVES - 1) run += seg_sum[w];
    }
    while (owner > 0 && owner * seg >= vocab) --owner;    // never an empty segment
    owner_s = owner;
    walk[0] = run;
    walk[1] = target;
  }
  __syncthreads();
  if (wave != owner_s) return;
  // ---- the owner walks its segment in index order, 64 tokens at a time, with a prefix sum over lanes
  float run = walk[0];
  const float target = walk[1];
  int pick = se - 1;                       // if rounding leaves the target just past the segment's mass
  for (int base = sb; base < se; base += WAVE) {
    const int i = base + lane;
    float e = i < se ? __expf((x[i] - mx) * inv_t) : 0.f;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {   // inclusive prefix sum
      const float up = __shfl_up(e, o, WAVE);
      if (lane >= o) e += up;
    }
    const unsigned long long hit = __ballot(run + e > target && i < se);
    if (hit) {
      pick = base + __ffsll((long long)hit) - 1;
      break;
    }
    run += __shfl(e, WAVE - 1, WAVE);
  }
  if (lane == 0) out[r] = pick;
}

// out: [R] int32; logits: [R, vocab] float with row stride; temperature, uniform: [R] float
// (temperature may be null: all rows greedy).
extern "C" int ga_sample_rows(void* out, const void* logits, int64_t row_stride, int rows, int vocab,
                              const void* temperature, const void* uniform, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return -1;
  hipLaunchKernelGGL(sample_rows_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, (int32_t*)out,
                     (const float*)logits, row_stride, vocab, (const float*)temperature,
                     (const float*)uniform);
  return GA_CHECK_LAUNCH();
}
