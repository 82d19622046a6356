// Seeded normal fill on the host: the same element values as the device kernel (../counter_normal.h),
// so that a model folder written here and a model made in device memory from the same seed hold the same
// weights.  Threads split the tensor into contiguous ranges; every element depends on (seed, index) only.
#include <stddef.h>
#include <stdint.h>

#include <algorithm>
#include <thread>
#include <vector>

#include "../counter_normal.h"

namespace {

// float32 -> bfloat16, round to nearest, ties to even; NaN stays NaN (the kernels' conversion)
inline uint16_t to_bf16_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

void fill_range(void* out, int dtype, size_t lo, size_t hi, uint64_t seed, double mean, double std) {
  if (dtype == 0) {
    float* p = (float*)out;
    for (size_t i = lo; i < hi; ++i) p[i] = cn_element(seed, i, mean, std);
  } else {
    uint16_t* p = (uint16_t*)out;
    for (size_t i = lo; i < hi; ++i) p[i] = to_bf16_bits(cn_element(seed, i, mean, std));
  }
}

}  // namespace

// dtype: 0 float32, 1 bfloat16 (the kernel library's codes).  Returns 0, or 1 for an unknown dtype.
extern "C" int hr_fill_normal(void* out, int dtype, size_t n, unsigned long long seed, double mean, double std,
                              int threads) {
  if (dtype != 0 && dtype != 1) return 1;
  if (n == 0) return 0;
  const size_t per_thread_min = 1 << 16;
  size_t nt = std::max<size_t>(1, std::min<size_t>((size_t)std::max(1, threads), (n + per_thread_min - 1) / per_thread_min));
  if (nt == 1) {
    fill_range(out, dtype, 0, n, seed, mean, std);
    return 0;
  }
  std::vector<std::thread> pool;
  const size_t chunk = (n + nt - 1) / nt;
  for (size_t t = 0; t < nt; ++t) {
    const size_t lo = t * chunk, hi = std::min(n, lo + chunk);
    if (lo >= hi) break;
    pool.emplace_back(fill_range, out, dtype, lo, hi, (uint64_t)seed, mean, std);
  }
  for (auto& th : pool) th.join();
  return 0;
}
