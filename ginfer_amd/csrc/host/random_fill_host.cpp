// The host's side of the random-weights generator: the same function of (key, element) as the device kernel in
// random_fill.hip (both include random_normal.h), over a few threads.  Plain C++, no GPU runtime: it writes model
// folders on machines without a GPU.
#include "../random_normal.h"

#include <thread>
#include <vector>

extern "C" int ga_random_normal_fill_host(float* out, int64_t n, uint64_t key, float mean, float std, int threads) {
  if (n <= 0) return 0;
  if (!out) return -1;
  if (threads < 1) threads = 1;
  if (threads > 64) threads = 64;
  if (n < (int64_t)1 << 16) threads = 1;
  std::vector<std::thread> pool;
  const int64_t per = (n + threads - 1) / threads;
  for (int t = 0; t < threads; ++t) {
    const int64_t begin = t * per, end = begin + per < n ? begin + per : n;
    if (begin >= end) break;
    pool.emplace_back([=]() {
      for (int64_t i = begin; i < end; ++i) out[i] = ga_weight_from_counter(key, (uint64_t)i, mean, std);
    });
  }
  for (auto& th : pool) th.join();
  return 0;
}
