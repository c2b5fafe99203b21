// Fused residual add + RMSNorm.
//   h = residual[t] + delta[t]        (32-bit add; written back to the 32-bit residual stream)
//   y = (h * g) / sqrt(sum(h^2)/H + eps)
// Formula and order of operations: ginfer/core/op/kernels/cuda/rmsnorm_kernel.cu:27-66 (sum :31-44,
// rms :54, (x*g)/rms :63); the add replaces ginfer/core/op/kernels/cuda/add_kernel.cu:10-35, which
// adds in 16-bit.  With `rows` the kernel normalises only the listed rows (the gather before the
// output head, ginfer/core/op/kernels/cuda/select_last_token_kernel.cu:8-27) and leaves the
// residual stream untouched, so a row may be listed twice.
// The sum over a row is taken in a fixed order that depends on H alone, so a row's result does not
// depend on which other rows are in the batch.
#include "common.cuh"

#define NORM_THREADS 256

// D is the type of delta: the compute dtype, or float when delta holds `parts` partial sums of a
// K-split matrix product ([parts][T][H]); the parts are added in order, after one another.
template <typename T, typename G, typename D>
__global__ void add_rmsnorm_kernel(T* __restrict__ out, float* __restrict__ residual,
                                   const D* __restrict__ delta, int parts, int64_t part_stride,
                                   const G* __restrict__ gain, const int32_t* __restrict__ rows, int hidden,
                                   float eps) {
  __shared__ float scratch[NORM_THREADS / WAVE];
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? (int64_t)rows[r] : r;
  float* res = residual + t * hidden;
  const D* d = delta ? delta + t * hidden : nullptr;
  const bool write_back = (rows == nullptr) && (d != nullptr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += NORM_THREADS) {
    float h = res[i];
    if (d) {
      float add = Num<D>::ld(d + i);
      for (int p = 1; p < parts; ++p) add += Num<D>::ld(d + p * part_stride + i);
      h += add;
    }
    if (write_back) res[i] = h;
    ss += h * h;
  }
  ss = block_sum<NORM_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps);
  T* o = out + r * hidden;
  for (int i = threadIdx.x; i < hidden; i += NORM_THREADS) {
    float h = res[i];                       // own write of the first pass when write_back
    if (d && !write_back) {
      float add = Num<D>::ld(d + i);
      for (int p = 1; p < parts; ++p) add += Num<D>::ld(d + p * part_stride + i);
      h += add;
    }
    Num<T>::st(o + i, (h * Num<G>::ld(gain + i)) / rms);
  }
}

// out: [R, H] in the compute dtype; residual: [T, H] float; delta: [T, H] compute dtype or null, or, with
// delta_parts > 0, float [delta_parts][T][H] partial sums; gain: [H] compute dtype, or float when
// gain_is_f32; rows: [R] int32 or null (then R == T); num_tokens = T.
extern "C" int ga_add_rmsnorm(void* out, void* residual, const void* delta, int delta_parts, int num_tokens,
                              const void* gain, const void* rows, int num_rows, int hidden, float eps,
                              int is_bf16, int gain_is_f32, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  dim3 grid(num_rows), block(NORM_THREADS);
  const int64_t stride = (int64_t)num_tokens * hidden;
#define LAUNCH(T, G, D, PARTS)                                                                    \
  hipLaunchKernelGGL((add_rmsnorm_kernel<T, G, D>), grid, block, 0, stream, (T*)out,             \
                     (float*)residual, (const D*)delta, PARTS, stride, (const G*)gain,            \
                     (const int32_t*)rows, hidden, eps)
  if (delta_parts > 0) {
    if (is_bf16) {
      if (gain_is_f32) LAUNCH(bf16_t, float, float, delta_parts); else LAUNCH(bf16_t, bf16_t, float, delta_parts);
    } else {
      LAUNCH(float, float, float, delta_parts);
    }
  } else if (is_bf16) {
    if (gain_is_f32) LAUNCH(bf16_t, float, bf16_t, 1); else LAUNCH(bf16_t, bf16_t, bf16_t, 1);
  } else {
    LAUNCH(float, float, float, 1);
  }
#undef LAUNCH
  return GA_CHECK_LAUNCH();
}
