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

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(
    int32_t* __restrict__ out, const float* __restrict__ logits, int64_t row_stride, int vocab,
    const float* __restrict__ temperature, const float* __restrict__ uniform) {
  __shared__ float part_f[SAMPLE_THREADS];
  __shared__ int part_i[SAMPLE_THREADS];
  __shared__ int chosen;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (int64_t)r * row_stride;
  // contiguous chunk per thread, so that index order is thread order
  const int chunk = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int begin = tid * chunk < vocab ? tid * chunk : vocab;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;

  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = begin; i < end; ++i) {
    const float v = x[i];
    if (best_i == 0x7fffffff || v > best) { best = v; best_i = i; }   // strictly greater: lowest index wins
  }
  part_f[tid] = best;
  part_i[tid] = best_i;
  __syncthreads();
  for (int s = SAMPLE_THREADS / 2; s > 0; s >>= 1) {
    if (tid < s) {
      const float a = part_f[tid], b = part_f[tid + s];
      const int ai = part_i[tid], bi = part_i[tid + s];
      // among equal values the lower index wins (the two halves interleave index ranges)
      if (bi != 0x7fffffff && (ai == 0x7fffffff || b > a || (b == a && bi < ai))) {
        part_f[tid] = b;
        part_i[tid] = bi;
      }
    }
    __syncthreads();
  }
  const float mx = part_f[0];
  const int arg = part_i[0];
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = arg;
    return;
  }
  __syncthreads();
  const float inv_t = 1.0f / temp;
  float sum = 0.f;
  for (int i = begin; i < end; ++i) sum += expf((x[i] - mx) * inv_t);
  part_f[tid] = sum;
  if (tid == 0) chosen = -1;
  __syncthreads();
  if (tid == 0) {
    // serial scan over the thread sums: 1024 additions, in index order
    float total = 0.f;
    for (int i = 0; i < SAMPLE_THREADS; ++i) total += part_f[i];
    const float target = uniform[r] * total;
    float run = 0.f;
    int owner = -1;
    for (int i = 0; i < SAMPLE_THREADS; ++i) {
      if (run + part_f[i] > target) { owner = i; break; }
      run += part_f[i];
    }
    part_i[0] = owner;
    part_f[0] = run;          // mass before the owner's chunk (the owner's own sum is not needed)
    part_f[1] = target;
  }
  __syncthreads();
  const int owner = part_i[0];
  if (owner < 0) {            // rounding pushed the target past the end: the last index with mass
    if (tid == 0) out[r] = vocab - 1;
    return;
  }
  if (tid == owner) {
    float run = part_f[0];
    const float target = part_f[1];
    int pick = end - 1;
    for (int i = begin; i < end; ++i) {
      run += expf((x[i] - mx) * inv_t);
      if (run > target) { pick = i; break; }
    }
    out[r] = pick;
  }
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
