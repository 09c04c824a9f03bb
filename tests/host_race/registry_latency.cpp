// Registry latency at the size of benchmark configuration 4: 100,000 tracked entries (its sub-allocation
// count) are added through the allocator hook, looked up by handle and by address, and deleted again,
// and the time per call is printed. Registry only: made-up addresses, no GPU, no peer service.
#include <stdio.h>
#include <stdlib.h>

#include <chrono>
#include <vector>

#include "../../include/amem.h"

using Clock = std::chrono::steady_clock;
static double us_per(Clock::time_point t0, size_t n) {
  return std::chrono::duration<double, std::micro>(Clock::now() - t0).count() / (double)n;
}

int main(int argc, char** argv) {
  const size_t N = argc > 1 ? (size_t)atol(argv[1]) : 100000;
  if (amem_set_enabled(1) != 0) return 1;
  // sizes log-uniform in [4, 64) KiB like the configuration's, bump-allocated addresses
  std::vector<uint64_t> va(N), handle(N), size(N);
  uint64_t x = 88172645463325252ull, cur = 0x7e0000000000ull;
  for (size_t i = 0; i < N; ++i) {
    x ^= x << 13; x ^= x >> 7; x ^= x << 17;
    size[i] = (4096ull << (x % 4)) + ((x >> 8) % (4096ull << (x % 4))) / 4096 * 4096;
    va[i] = cur;
    cur += size[i];
    handle[i] = 0x100000000ull + i * 16;
  }
  // registration order is not address order in real life: shuffle
  std::vector<size_t> order(N);
  for (size_t i = 0; i < N; ++i) order[i] = i;
  for (size_t i = N - 1; i > 0; --i) { x ^= x << 13; x ^= x >> 7; x ^= x << 17; std::swap(order[i], order[x % (i + 1)]); }
  long bad = 0;
  auto t0 = Clock::now();
  for (size_t k = 0; k < N; ++k) {
    const size_t i = order[k];
    bad += amem_add_alloc_info(va[i], size[i], AMEM_TYPE_LOCAL, 0, handle[i], -1, 0, nullptr, (int)(i % 8)) != 0;
  }
  const double add_us = us_per(t0, N);
  bad += amem_region_count(0) != (int64_t)N;
  t0 = Clock::now();
  for (size_t k = 0; k < N; ++k) bad += amem_handle_lookup(0, handle[order[k]]) != va[order[k]];
  const double lookup_us = us_per(t0, N);
  amem_region_info info;
  t0 = Clock::now();
  for (size_t k = 0; k < N; ++k) bad += amem_region_find(0, va[order[k]], &info) != 0 || info.alloc_sz != size[order[k]];
  const double find_us = us_per(t0, N);
  t0 = Clock::now();
  for (size_t k = 0; k < N; ++k) bad += amem_check_paused(0) != 0;
  const double gate_us = us_per(t0, N);
  t0 = Clock::now();
  for (size_t k = 0; k < N; ++k) bad += amem_del_alloc_info(va[order[k]], handle[order[k]], 0) != 0;
  const double del_us = us_per(t0, N);
  bad += amem_region_count(0) != 0 || amem_handle_count(0) != 0;
  amem_counters c;
  amem_get_counters(&c);
  for (int i = 0; i < AMEM_MAX_CALLER; ++i) bad += c.alloc_bytes[i] != 0;
  printf("registry latency, %zu entries: add %.3f us, lookup by handle %.3f us, find by address %.3f us, "
         "paused gate %.3f us, delete %.3f us per call; errors %ld\n", N, add_us, lookup_us, find_us, gate_us, del_us, bad);
  return bad ? 1 : 0;
}
