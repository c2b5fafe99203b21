// Choosing the next token from 32-bit logits in two launches: every row's vocabulary is cut into
// segments that workgroups scan side by side, then one workgroup per row picks.
//   temperature == 0: argmax, the lowest index among equal maxima (the reference's reduction,
//     ginfer/core/op/kernels/cuda/argmax_kernel.cu:52-98, keeps whichever equal value its tree meets
//     first; ginfer/model/model.cc:219-220 is where it is used).
//   temperature  > 0: p = softmax(logits / temperature) in 32-bit, and the first index whose running
//     sum of exp((x - max) / temperature) exceeds uniform * total: an inverse-CDF draw from a uniform
//     number the caller supplies, so the choice is a pure function of (logits, temperature, uniform):
//     the cut into segments depends on the vocabulary alone, never on the rows beside it.
// The reference samples greedily only (ginfer/engine/sampling_params.h:5-8).
#include "common.h"
#include "ginfer_amd.h"   // the entry points below are checked against their declarations
#include <atomic>
#include <mutex>

#define SCAN_THREADS 256
#define SCAN_WAVES (SCAN_THREADS / WAVE)
#define MAX_SEGMENTS 64
#define NO_INDEX 0x7fffffff

__device__ __forceinline__ bool better(float b, int bi, float best, int best_i) {
  return bi != NO_INDEX && (best_i == NO_INDEX || b > best || (b == best && bi < best_i));
}

// Segment (blockIdx.x) of row (blockIdx.y): its maximum with the lowest index that holds it, and, for a
// row with a temperature, the sum of exp((x - segment max) / temperature) over the segment.
__global__ __launch_bounds__(SCAN_THREADS) void sample_scan_kernel(
    float* __restrict__ seg_max, int32_t* __restrict__ seg_arg, float* __restrict__ seg_sum,
    const float* __restrict__ logits, int64_t row_stride, int vocab, int seg, int segments,
    const float* __restrict__ temperature) {
  __shared__ float part_f[SCAN_WAVES];
  __shared__ int part_i[SCAN_WAVES];
  const int s = blockIdx.x, r = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const float* x = logits + (int64_t)r * row_stride;
  const int sb = s * seg < vocab ? s * seg : vocab;
  const int se = sb + seg < vocab ? sb + seg : vocab;
  // strided (coalesced) reads, four loads in flight; a thread meets its indices in ascending order
  float bests[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
  int bests_i[4] = {NO_INDEX, NO_INDEX, NO_INDEX, NO_INDEX};
  for (int i0 = sb + tid; i0 < se; i0 += 4 * SCAN_THREADS) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * SCAN_THREADS;
      v[u] = i < se ? x[i] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * SCAN_THREADS;
      if (i < se && (bests_i[u] == NO_INDEX || v[u] > bests[u])) { bests[u] = v[u]; bests_i[u] = i; }
    }
  }
  float best = bests[0];
  int best_i = bests_i[0];
#pragma unroll
  for (int u = 1; u < 4; ++u)
    if (better(bests[u], bests_i[u], best, best_i)) { best = bests[u]; best_i = bests_i[u]; }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float b = __shfl_xor(best, o, WAVE);
    const int bi = __shfl_xor(best_i, o, WAVE);
    if (better(b, bi, best, best_i)) { best = b; best_i = bi; }
  }
  if (lane == 0) { part_f[wave] = best; part_i[wave] = best_i; }
  __syncthreads();
  float mx = part_f[0];
  int arg = part_i[0];
#pragma unroll
  for (int w = 1; w < SCAN_WAVES; ++w)
    if (better(part_f[w], part_i[w], mx, arg)) { mx = part_f[w]; arg = part_i[w]; }
  const int64_t o = (int64_t)r * segments + s;
  if (tid == 0) { seg_max[o] = mx; seg_arg[o] = arg; }
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) return;
  const float inv_t = 1.0f / temp;
  float sum = 0.f;
  for (int i = sb + tid; i < se; i += SCAN_THREADS) sum += __expf((x[i] - mx) * inv_t);
  sum = block_sum<SCAN_WAVES>(sum, part_f);
  if (tid == 0) seg_sum[o] = sum;
}

// One workgroup per row: the row's maximum from the segments' (lowest segment first, so the lowest index
// wins among equals); with a temperature, the segments' masses brought to the row's maximum, added in
// segment order, the segment that holds uniform * total, and inside it SCAN_THREADS runs of consecutive
// tokens whose masses are added in order until the target is passed.
__global__ __launch_bounds__(SCAN_THREADS) void sample_pick_kernel(
    int32_t* __restrict__ out, const float* __restrict__ seg_max, const int32_t* __restrict__ seg_arg,
    const float* __restrict__ seg_sum, const float* __restrict__ logits, int64_t row_stride, int vocab, int seg,
    int segments, const float* __restrict__ temperature, const float* __restrict__ uniform) {
  __shared__ float mass[MAX_SEGMENTS];
  __shared__ float runs[SCAN_THREADS];
  __shared__ float walk[3];
  __shared__ int owner_s[2];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (int64_t)r * row_stride;
  const int64_t o = (int64_t)r * segments;
  float mx = seg_max[o];
  int arg = seg_arg[o];
  for (int s = 1; s < segments; ++s)
    if (better(seg_max[o + s], seg_arg[o + s], mx, arg)) { mx = seg_max[o + s]; arg = seg_arg[o + s]; }
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = arg;
    return;
  }
  const float inv_t = 1.0f / temp;
  if (tid < segments) mass[tid] = seg_sum[o + tid] * __expf((seg_max[o + tid] - mx) * inv_t);
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int s = 0; s < segments; ++s) total += mass[s];
    const float target = uniform[r] * total;
    float run = 0.f;
    int owner = segments - 1;
    for (int s = 0; s < segments; ++s) {
      if (run + mass[s] > target) { owner = s; break; }
      if (s < segments - 1) run += mass[s];
    }
    while (owner > 0 && owner * seg >= vocab) --owner;    // never an empty segment
    owner_s[0] = owner;
    walk[0] = run;
    walk[1] = target;
  }
  __syncthreads();
  const int owner = owner_s[0];
  const float target = walk[1];
  const int sb = owner * seg, se = sb + seg < vocab ? sb + seg : vocab;
  const int per = (se - sb + SCAN_THREADS - 1) / SCAN_THREADS;     // consecutive tokens of a thread
  const int tb = sb + tid * per < se ? sb + tid * per : se;
  const int te = tb + per < se ? tb + per : se;
  float mine = 0.f;
  for (int i = tb; i < te; ++i) mine += __expf((x[i] - mx) * inv_t);
  runs[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float run = walk[0];
    int t = SCAN_THREADS - 1;
    for (int k = 0; k < SCAN_THREADS; ++k) {
      if (run + runs[k] > target) { t = k; break; }
      if (k < SCAN_THREADS - 1) run += runs[k];
    }
    while (t > 0 && sb + t * per >= se) --t;                // never an empty run
    owner_s[1] = t;
    walk[2] = run;
  }
  __syncthreads();
  if (tid != owner_s[1]) return;
  float run = walk[2];
  int pick = te - 1;                       // if rounding leaves the target just past the run's mass
  for (int i = tb; i < te; ++i) {
    run += __expf((x[i] - mx) * inv_t);
    if (run > target) { pick = i; break; }
  }
  out[r] = pick;
}

// How the vocabulary is cut: a function of its size alone.
static void segments_of(int vocab, int* seg, int* segments) {
  int n = (vocab + 2047) / 2048;
  if (n > MAX_SEGMENTS) n = MAX_SEGMENTS;
  if (n < 1) n = 1;
  *seg = (vocab + n - 1) / n;
  *segments = (vocab + *seg - 1) / *seg;
}

// Floats of scratch memory that ga_sample_rows needs for these sizes.
extern "C" int64_t ga_sample_scratch_floats(int rows, int vocab) {
  int seg, segments;
  segments_of(vocab > 0 ? vocab : 1, &seg, &segments);
  return (int64_t)3 * (rows > 0 ? rows : 0) * segments;
}

// out: [R] int32; logits: [R, vocab] float with row stride; temperature, uniform: [R] float
// (temperature may be null: all rows greedy); scratch: ga_sample_scratch_floats(rows, vocab) floats.
extern "C" int ga_sample_rows(void* out, const void* logits, int64_t row_stride, int rows, int vocab,
                              const void* temperature, const void* uniform, void* scratch, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || !scratch) return -1;
  int seg, segments;
  segments_of(vocab, &seg, &segments);
  float* seg_max = (float*)scratch;
  int32_t* seg_arg = (int32_t*)(seg_max + (int64_t)rows * segments);
  float* seg_sum = seg_max + (int64_t)2 * rows * segments;
  hipLaunchKernelGGL(sample_scan_kernel, dim3(segments, rows), dim3(SCAN_THREADS), 0, stream, seg_max, seg_arg,
                     seg_sum, (const float*)logits, row_stride, vocab, seg, segments, (const float*)temperature);
  hipLaunchKernelGGL(sample_pick_kernel, dim3(rows), dim3(SCAN_THREADS), 0, stream, (int32_t*)out, seg_max,
                     seg_arg, seg_sum, (const float*)logits, row_stride, vocab, seg, segments,
                     (const float*)temperature, (const float*)uniform);
  return GA_CHECK_LAUNCH();
}

// ---- the same choice for callers that cannot allocate
//
// ga_sample_rows takes its scratch memory from the caller, who has to allocate it.  Code that runs under HIP
// graph capture, a tight serving loop or a harness that forbids allocation cannot: for them the scratch lies in
// a file-scope device array of a fixed, modest size, which every GPU that this library runs on holds until the
// process ends (STATIC_SCRATCH_FLOATS * 4 = 196,608 bytes).  In host code the array's name stands for the symbol,
// not for device memory: its address on a device is looked up once per device (hipGetSymbolAddress, with that
// device current) and only that address is ever handed to a kernel.
#define STATIC_MAX_ROWS 256
#define STATIC_SCRATCH_FLOATS (3 * STATIC_MAX_ROWS * MAX_SEGMENTS)
#define STATIC_MAX_DEVICES 64
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

static std::mutex scratch_lock;
static std::atomic<float*> scratch_on_device[STATIC_MAX_DEVICES];   // the array's address on each device, once known

// The address of `scratch` on the current device, looked up at the first call on that device; null (and *rc set)
// if the runtime refuses.
static float* static_scratch(int* rc) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) { *rc = (int)e; return nullptr; }
  if (device < 0 || device >= STATIC_MAX_DEVICES) { *rc = -3; return nullptr; }
  float* p = scratch_on_device[device].load(std::memory_order_acquire);
  if (p) return p;
  std::lock_guard<std::mutex> hold(scratch_lock);
  p = scratch_on_device[device].load(std::memory_order_acquire);
  if (p) return p;
  void* address = nullptr;
  e = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !address) { *rc = e != hipSuccess ? (int)e : -4; return nullptr; }
  p = (float*)address;
  scratch_on_device[device].store(p, std::memory_order_release);
  return p;
}

// Rows that ga_sample_rows_static takes in one call.
extern "C" int ga_sample_rows_static_max_rows() { return STATIC_MAX_ROWS; }

// Looks up the scratch array on the current device, so that the first ga_sample_rows_static there does nothing
// but launch (a caller that is about to record a graph calls this before).  0, or the runtime's error code.
extern "C" int ga_sample_rows_static_init() {
  int rc = 0;
  return static_scratch(&rc) ? 0 : rc;
}

// What a negative return value of ga_sample_rows_static means.
extern "C" const char* ga_sample_rows_static_error(int code) {
  switch (code) {
    case 0: return "ok";
    case -1: return "vocab must be positive";
    case -2: return "more rows than ga_sample_rows_static_max_rows(): the static scratch array holds 256 rows";
    case -3: return "the current device's number is beyond the devices this library keeps an address for (64)";
    case -4: return "the scratch array has no address on the current device";
    default: return code > 0 ? "an error code of the HIP runtime" : "unknown";
  }
}

// ga_sample_rows without a scratch argument and without any allocation: the segments' results go through the
// static array.  At most ga_sample_rows_static_max_rows() rows a call (more: -2, nothing launched).  Every call
// on a GPU shares that GPU's array: calls that overlap there (two streams, two threads) race; calls in one stream
// do not.  Nothing in the array has to start at zero: the first kernel writes every word the second one reads.
extern "C" int ga_sample_rows_static(void* out, const void* logits, int64_t row_stride, int rows, int vocab,
                                     const void* temperature, const void* uniform, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return -1;
  if (rows > STATIC_MAX_ROWS) return -2;
  int rc = 0;
  float* ptr = static_scratch(&rc);
  if (!ptr) return rc;
  return ga_sample_rows(out, logits, row_stride, rows, vocab, temperature, uniform, ptr, stream);
}
