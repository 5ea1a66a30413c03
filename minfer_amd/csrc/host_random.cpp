// Host side of the seeded normal fill: the same values as `fill_normal_kernel` in
// elementwise.hip produces on the GPU (both call mf_normal_value of random_normal.h), written
// into host memory by a few threads.  Compiled with the host compiler only; nothing here touches
// the GPU.
#include <stddef.h>
#include <stdint.h>

#include <thread>
#include <vector>

#include "random_normal.h"

extern "C" __attribute__((visibility("default"))) int mf_fill_normal_host(void* out, int is_bf16, size_t n,
                                                                          uint64_t seed, float std,
                                                                          int round_bf16, int n_threads) {
  if (n == 0) return 0;
  if (!out || n_threads < 1) return 1;
  auto work = [=](size_t begin, size_t end) {
    // whole pairs: `begin` is even
    for (size_t i = begin; i < end; i += 2) {
      double z0, z1;
      mf_normal_pair(seed, i >> 1, &z0, &z1);
      const float v0 = (float)z0 * std, v1 = (float)z1 * std;
      if (is_bf16) {
        uint16_t* o = (uint16_t*)out;
        o[i] = mf_bf16_bits(v0);
        if (i + 1 < end) o[i + 1] = mf_bf16_bits(v1);
      } else {
        float* o = (float*)out;
        o[i] = round_bf16 ? mf_bf16_value(mf_bf16_bits(v0)) : v0;
        if (i + 1 < end) o[i + 1] = round_bf16 ? mf_bf16_value(mf_bf16_bits(v1)) : v1;
      }
    }
  };
  const size_t pairs = (n + 1) / 2;
  size_t threads = (size_t)n_threads;
  if (pairs < 4096 * threads) threads = pairs / 4096 ? pairs / 4096 : 1;
  std::vector<std::thread> pool;
  const size_t per = (pairs + threads - 1) / threads;
  for (size_t t = 0; t < threads; ++t) {
    const size_t b = t * per * 2, e = (t + 1) * per * 2 < n ? (t + 1) * per * 2 : n;
    if (b >= n) break;
    if (t + 1 == threads || e == n) {
      work(b, n);
      break;
    }
    pool.emplace_back(work, b, e);
  }
  for (auto& th : pool) th.join();
  return 0;
}
